"""GPU op-test command lines (tests/cpp), the counterparts of the reference's
op_test_flash_attn / op_test_rope_single binaries, and the AttentionGPUImpl layer
driven through prefill + decode steps.  They go through the C++ device layer
(Tensor, GPUAllocator, hip_ops.hpp) on top of the C ABI."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "bin")


def _run(exe, *flags):
    print("running", exe, *flags, flush=True)
    r = subprocess.run([os.path.join(BIN, exe), *map(str, flags)], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and ("PASS" in r.stdout or "test success" in r.stdout), r.stdout + r.stderr
    return r.stdout


@pytest.mark.parametrize("flags", [
    ("--m", 256, "--n", 256, "--offset", 0, "--head_num", 32, "--head_dim", 128),                 # benchmark configuration 1
    ("--m", 1, "--n", 512, "--offset", 511, "--head_num", 32),                                    # config 2
    ("--m", 256, "--n", 256, "--head_num", 12, "--kv_head_num", 2, "--dtype", "bf16"),            # config 3 prefill
    ("--m", 1024, "--n", 1024, "--head_num", 28, "--kv_head_num", 4, "--dtype", "bf16"),          # config 4, S=1024
    ("--m", 100, "--n", 612, "--offset", 512, "--head_num", 8, "--kv_head_num", 8),               # chunked prefill
])
def test_op_test_flash_attn(flags):
    _run("op_test_flash_attn", *flags)


@pytest.mark.parametrize("flags", [
    ("--dtype", "fp16", "--is_neox", 0, "--offset", 0, "--seq_len", 128),
    ("--dtype", "fp16", "--is_neox", 1, "--offset", 1000, "--seq_len", 77),
    ("--dtype", "bf16", "--is_neox", 1, "--offset", 511, "--seq_len", 1, "--theta", 1000000, "--head_num", 12),
    ("--dtype", "bf16", "--is_neox", 0, "--offset", 5, "--seq_len", 300, "--head_num", 2),
])
def test_op_test_rope_single(flags):
    _run("op_test_rope_single", *flags)


@pytest.mark.parametrize("flags", [
    ("--head_num", 12, "--kv_head_num", 2, "--prompt", 256, "--steps", 24, "--dtype", "bf16", "--is_neox", 1),  # config 3
    ("--head_num", 32, "--kv_head_num", 32, "--prompt", 40, "--steps", 6, "--dtype", "fp16", "--is_neox", 0,
     "--theta", 10000),
    # chunked prefill through the layer: 64 more tokens over a 2403-row cache (key-range split, packed rows)
    ("--head_num", 28, "--kv_head_num", 4, "--prompt", 2400, "--steps", 3, "--chunk", 64, "--max_seq_len", 2560,
     "--dtype", "bf16", "--is_neox", 1),
])
def test_attention_layer_prefill_then_decode(flags):
    _run("op_test_attention_layer", *flags)


@pytest.mark.parametrize("flags", [
    # Llama2-7B, benchmark configurations 1 and 2 in one run: prefill 256, decode up to row 511
    ("--model", "llama2", "--head_num", 32, "--kv_head_num", 32, "--prompt", 256, "--steps", 12, "--dtype", "fp16",
     "--is_neox", 0, "--theta", 10000, "--max_seq_len", 512),
    ("--model", "llama2", "--head_num", 8, "--kv_head_num", 8, "--prompt", 100, "--steps", 4, "--chunk", 40,
     "--dtype", "bf16", "--is_neox", 1, "--max_seq_len", 256),
])
def test_llama_sequence_through_the_device_switch(flags):
    """Llama2AttentionLayer (DEV_GPU arm of the layer switch): RoPELayer::Forward -> two device-to-device copies
    -> hip_flash_attn_opt_prefill_layer, as src/llama2_layer_npu.cpp:284, :325-339, :370-374 issues them;
    outputs and caches bit-identical to the fused path, and within tolerance of the oracle."""
    out = _run("op_test_attention_layer", *flags)
    assert "vs fused path: outputs bit-identical" in out and "caches bit-identical" in out, out


def test_qwen_layer_through_the_device_switch_and_decode_loop_timing():
    """Qwen2AttentionLayer behind the facade, checked; then the decode loop of benchmark configuration 3
    (256 prompt tokens, 256 generated) timed through the layer: no host wait per step, no event of the pool."""
    import json
    _run("op_test_attention_layer", "--model", "qwen2", "--head_num", 12, "--kv_head_num", 2, "--prompt", 256,
         "--steps", 16, "--dtype", "bf16", "--is_neox", 1)
    exe = os.path.join(BIN, "op_test_attention_layer")
    r = subprocess.run([exe, "--head_num", "12", "--kv_head_num", "2", "--prompt", "256", "--steps", "256",
                        "--time", "3", "--dtype", "bf16"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    t = json.loads(r.stdout.strip().splitlines()[-1])
    print(t, flush=True)
    assert t["status"] == 0 and t["pool_fence_events"] == 0
    assert 0 < t["layer_decode_us_per_step"] < 200 and 0 < t["abi_decode_us_per_step"] < 200


def test_stream_ordered_pool_on_the_device():
    """A block freed under queued work goes back to its own stream at once, to another stream or to host code only
    after that work is done; the kernel that was reading it produces the right output."""
    out = _run("op_test_pool")
    assert "pointers as expected" in out, out


@pytest.mark.parametrize("flags", [
    ("--m", 2048, "--n", 2048, "--k", 2048, "--dtype", "fp16"),                       # the reference CLI's defaults
    ("--m", 256, "--n", 3584, "--k", 3584, "--bias", 1, "--dtype", "bf16"),           # Qwen2.5-7B q_proj
    ("--m", 1, "--n", 512, "--k", 3584, "--bias", 1, "--dtype", "bf16"),              # k_proj, decode
])
def test_op_test_gemm(flags):
    _run("op_test_gemm", *flags)


@pytest.mark.parametrize("flags", [
    ("--head_num", 12, "--kv_head_num", 2, "--prompt", 256, "--steps", 6, "--dtype", "bf16"),     # Qwen2.5-1.5B shape
    ("--head_num", 28, "--kv_head_num", 4, "--prompt", 512, "--steps", 2, "--dtype", "bf16",
     "--max_seq_len", 1024),                                                                      # Qwen2.5-7B shape
    ("--head_num", 8, "--kv_head_num", 8, "--prompt", 40, "--steps", 3, "--dtype", "fp16", "--is_neox", 0,
     "--theta", 10000, "--bias", 0),                                                              # Llama-style
])
def test_attention_block_with_projections_and_trace(flags, tmp_path):
    """q/k/v projections -> RoPE + append -> attention -> o_proj -> residual add, profiled: the
    trace file must be the Chrome-trace JSON the reference's profiler writes
    (src/profiling.cpp:11-38, :80-93)."""
    import json
    trace = tmp_path / "trace.json"
    _run("op_test_attention_block", *flags, "--trace", trace)
    events = json.loads(trace.read_text())
    steps = flags[flags.index("--steps") + 1]
    assert len(events) == 6 * (steps + 1)
    names = [e["name"] for e in events[:6]]
    assert names == ["MatmulLayer"] * 3 + ["RoPE+KVAppend+FlashAttnGQA", "MatmulLayer", "Add"]
    for e in events:
        assert e["ph"] == "X" and e["pid"] == 0 and e["dur"] > 0 and e["ts"] >= 0
        assert set(e["args"]) == {"file", "lineno", "info"}
