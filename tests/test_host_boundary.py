"""CPU-side checks of the drop-in boundary: the shared library loads and exports
every symbol include/llmhip.h declares, arguments are validated before any launch,
and the C++ device layer (pooling allocator, Tensor, rotary table) behaves like the
reference's (src/device.hpp, src/device_npu.cpp).  No GPU needed, no compute calls."""
import ctypes
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_symbols(header="llmhip.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(llmhip_\w+)\s*\(", text))


def test_library_exports_every_declared_symbol():
    import llm_simple_amd.ops as ops
    declared = _header_symbols()
    assert declared == set(ops.SYMBOLS), declared ^ set(ops.SYMBOLS)
    handle = ctypes.CDLL(ops.LIB_PATH)
    for name in declared:
        assert hasattr(handle, name), name


def test_measurement_library_is_separate():
    """The measurement aids live in libllmhip_bench.so / llmhip_bench.h: the product library exports none
    of them, the measurement library exports exactly what its header declares, and validates arguments
    before touching a device."""
    import llm_simple_amd.bench_ops as bops
    import llm_simple_amd.ops as ops
    declared = _header_symbols("llmhip_bench.h")
    assert declared == set(bops.SYMBOLS), declared ^ set(bops.SYMBOLS)
    product = ctypes.CDLL(ops.LIB_PATH)
    for name in declared:
        assert hasattr(bops.lib, name), name
        assert not hasattr(product, name), name
    exported = subprocess.run(["nm", "-D", "--defined-only", ops.LIB_PATH], capture_output=True, text=True,
                              check=True).stdout
    assert "probe" not in exported and "clocked" not in exported and "ceiling" not in exported
    buf = ctypes.create_string_buffer(96)
    p = (ctypes.addressof(buf) + 15) & ~15
    # the plain-read probe: size a multiple of 16, sink of the declared size, aligned pointers
    assert bops.lib.llmhip_bench_stream_read(p, p, 24, p, bops.STREAM_READ_SINK_BYTES, 0, None) == -1
    assert bops.lib.llmhip_bench_stream_read(p, p, 32, p, 1024, 0, None) == -3
    assert bops.lib.llmhip_bench_stream_read(p, p + 4, 32, p, bops.STREAM_READ_SINK_BYTES, 0, None) == -1
    assert bops.lib.llmhip_bench_stream_read(p, p, 32, p, bops.STREAM_READ_SINK_BYTES, 2, None) == -1
    assert bops.lib.llmhip_bench_flash_attn_gqa_clocked(p, p, p, p, 1, 64, 63, 1, 1, 128, 5, p, None) == -2
    assert bops.lib.llmhip_bench_mfma_ceiling(2, 1.0, None) == -1


def test_cpp_overloads_cover_reference_operator_names():
    """hip_ops.hpp offers every attention / rope operator of prebuild/npu_ops.h:6-18, :39-47
    under the same name with the npu_ prefix replaced."""
    text = open(os.path.join(ROOT, "include", "hip_ops.hpp")).read()
    for name in ("hip_flash_attn_layer", "hip_flash_attn_gqa_layer", "hip_flash_attn_opt_prefill_layer",
                 "hip_rope_layer", "hip_rope_single_layer"):
        assert re.search(r"inline void %s\(" % name, text), name


def test_argument_validation_without_gpu():
    import llm_simple_amd.ops as ops
    buf = ctypes.create_string_buffer(96)
    p = (ctypes.addressof(buf) + 15) & ~15
    lib = ops.lib
    assert lib.llmhip_flash_attn(None, p, p, p, 1, 1, 0, 1, 128, 4, None) == -1
    assert lib.llmhip_flash_attn(p, p, p, p, 1, 1, 0, 1, 64, 4, None) == -2
    assert lib.llmhip_flash_attn_gqa(p, p, p, p, 1, 1, 0, 1, 1, 128, 7, None) == -1
    assert lib.llmhip_flash_decode_gqa(p, p, p, p, None, 0, 1, 4096, 4096, 5, 8, 128, 4, 5, None) == -3
    assert lib.llmhip_rope_single(p, p, p, 0, 1, 2, 100, 0, 4, None) == -2
    # misaligned device pointers are refused before any launch (the kernels move 16-byte pieces)
    assert p % 16 == 0
    assert lib.llmhip_flash_attn(p, p + 2, p, p, 1, 1, 0, 1, 128, 4, None) == -1
    assert lib.llmhip_flash_attn_gqa(p + 8, p, p, p, 1, 1, 0, 1, 1, 128, 4, None) == -1
    assert lib.llmhip_rope_single(p, p + 4, p, 0, 1, 2, 256, 0, 4, None) == -1
    assert lib.llmhip_rope_kv_append(p, p, p + 6, p, p, p, p, 0, 1, 1, 1, 128, 0, 4, None) == -1
    assert lib.llmhip_flash_decode_gqa_static(p, p, p + 2, p, 1, 16, 16, 5, 8, 128, 1, 5, None) == -1
    # the fused decode step: group size within the kernel's 16 columns, position not negative
    assert lib.llmhip_decode_step_gqa(p, p, p, p, p, p, p, 0, 17, 1, 128, 0, 5, None) == -2
    assert lib.llmhip_decode_step_gqa(p, p, p, p, p, p, p, -1, 5, 8, 128, 0, 5, None) == -1
    assert lib.llmhip_decode_step_gqa(p, p, p + 2, p, p, p, p, 0, 5, 8, 128, 0, 5, None) == -1
    try:
        ops.hip_flash_attn_layer(0, p, p, p, 1, 1, 0, 1, 128, 4)
    except ops.LlmHipError as e:
        assert e.status == -1 and "invalid" in str(e)
    else:
        raise AssertionError("expected LlmHipError")


def test_default_splits_and_workspace_size():
    import llm_simple_amd.ops as ops
    # about one workgroup per CU: batch * kv heads * splits ~ 256
    assert ops.flash_decode_default_splits(16, 32768, 8) == 2
    assert ops.flash_decode_default_splits(1, 32768, 8) == 32
    assert ops.flash_decode_default_splits(1, 64, 8) == 1
    s = ops.flash_decode_default_splits(1, 4096, 8)
    assert 1 <= s <= 32
    assert ops.flash_decode_workspace_bytes(1, 5, 8, 128, 1) == 0
    assert ops.flash_decode_workspace_bytes(16, 5, 8, 128, 2) == 16 * 8 * 2 * 16 * (128 + 2) * 4


def test_cpp_device_layer_host_checks():
    exe = os.path.join(ROOT, "tests", "cpp", "bin", "test_device_host")
    if not os.path.exists(exe):
        subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "tests", "cpp")])
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all passed" in r.stdout


def test_product_never_touches_the_oracle():
    """Nothing shipped imports, links or loads anything under oracle/."""
    pkg = os.path.join(ROOT, "llm_simple_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")) or f == "Makefile":
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)
    for f in ("llmhip.h", "hip_ops.hpp"):
        assert "oracle" not in open(os.path.join(ROOT, "include", f)).read().lower()


def test_default_workspace_size_covers_the_default_split_count():
    """num_splits <= 0 sizes the workspace for the largest count the default rule can pick, so a
    caller that lets the decode call choose never gets LLMHIP_ERR_WORKSPACE."""
    import llm_simple_amd.ops as ops
    for batch, hkv in ((1, 8), (16, 8), (3, 2), (1, 1), (64, 8), (20, 8), (24, 8), (40, 8), (48, 8), (12, 8), (7, 3)):
        cover = ops.flash_decode_workspace_bytes(batch, 5, hkv, 128, 0)
        for n in (1, 100, 129, 4096, 8192, 32768, 131072):
            s = ops.flash_decode_default_splits(batch, n, hkv)
            assert 1 <= s <= max(1, -(-n // 128)), (batch, hkv, n, s)  # every split holds at least one block
            assert ops.flash_decode_workspace_bytes(batch, 5, hkv, 128, s) <= cover, (batch, hkv, n)
    # the rule fills whole rounds of 256 workgroups where the pair count does not divide one
    assert ops.flash_decode_default_splits(40, 8192, 8) == 4    # 320 pairs -> 1280 workgroups = 5 rounds
    assert ops.flash_decode_default_splits(24, 8192, 8) == 4    # 192 pairs -> 768 = 3 rounds
    assert ops.flash_decode_default_splits(64, 4096, 8) == 1    # 512 pairs = 2 rounds already


def test_sanitizer_builds_of_oracle_and_device_layer():
    """Host-only -fsanitize=address,undefined builds: the CPU oracle driven over ragged shapes, and the
    C++ device layer with its injected allocator backend.  Both targets run what they build."""
    for sub in ("oracle", os.path.join("tests", "cpp")):
        r = subprocess.run(["make", "-s", "-C", os.path.join(ROOT, sub), "asan"], capture_output=True,
                           text=True, timeout=600)
        assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
        assert "ERROR: AddressSanitizer" not in r.stderr and "runtime error" not in r.stderr, r.stderr[-2000:]


def test_internal_scratch_size_of_the_reference_signature_calls():
    """Which llmhip_flash_attn* shapes take scratch from the per-stream buffer, and how much: none for square
    causal prefill, split-KV partials for decode-like shapes, key-range partials for a short chunk over a
    long cache (sized for the default 256 compute units when no GPU is visible)."""
    import llm_simple_amd.ops as ops
    f = ops.lib.llmhip_flash_attn_scratch_bytes
    for S in (256, 1024, 4096, 8192):
        assert f(S, S, 0, 7, 4) == 0            # Qwen2.5-7B prefill
    assert f(256, 256, 0, 1, 32) == 0           # Llama2-7B prefill
    assert f(1, 512, 511, 1, 32) == 32 * 4 * 16 * 130 * 4     # decode: 32 kv heads x 4 splits of 128 keys
    assert f(1, 32768, 32767, 5, 8) == ops.flash_decode_workspace_bytes(1, 5, 8, 128, 32)
    chunk = f(256, 33024, 32768, 7, 4)          # chunked prefill: 9 key ranges x 256 rows x 28 heads
    assert chunk == 9 * 256 * 28 * 130 * 4
    packed = f(40, 131072, 131032, 5, 8)        # 200 packed rows per kv head, 32 key ranges
    assert packed == 32 * 40 * 40 * 130 * 4
    assert f(0, 10, 0, 1, 1) == 0 and f(4, 0, 0, 1, 1) == 0   # invalid arguments
