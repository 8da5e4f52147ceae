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
    assert r.returncode == 0 and "PASS" in r.stdout, r.stdout + r.stderr
    return r.stdout


@pytest.mark.parametrize("flags", [
    ("--m", 256, "--n", 256, "--offset", 0, "--head_num", 32, "--head_dim", 128),                 # BASELINE config 1
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
])
def test_attention_layer_prefill_then_decode(flags):
    _run("op_test_attention_layer", *flags)
