"""ctypes binding of libllmhip_bench.so: the measurement aids of the benchmark
(include/llmhip_bench.h).  Not part of the product library; only bench.py and the tests of the
aids themselves import this module."""
import ctypes
import os

from . import ops

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libllmhip_bench.so")

_vp, _i, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
SYMBOLS = {
    "llmhip_bench_flash_attn_gqa_clocked": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _vp]),
    "llmhip_bench_mfma_ceiling": (_i, [_i, ctypes.c_double, ctypes.POINTER(ctypes.c_double)]),
    "llmhip_bench_stream_read": (_i, [_vp, _vp, _sz, _vp, _sz, _i, _vp]),
}


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is missing: build it with `make -C llm_simple_amd/csrc`")
    handle = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(handle, name)
        fn.restype = res
        fn.argtypes = args
    return handle


lib = _load()
STREAM_READ_SINK_BYTES = 65536


def _check(status, where):
    if status != 0:
        raise ops.LlmHipError(status, where)


def hip_flash_attn_gqa_clocked_layer(output_dev, q_dev, k_dev, v_dev, m, n, offset, group_size,
                                     kv_head_num, head_dim, dt, clock_probe_dev, stream=0):
    """hip_flash_attn_gqa_layer on the measurement library's copy of the prefill kernel, which also stores
    {shader-clock ticks, 100 MHz reference ticks} of its first workgroup at clock_probe_dev (two int64)."""
    p = ops._ptr
    _check(lib.llmhip_bench_flash_attn_gqa_clocked(p(output_dev), p(q_dev), p(k_dev), p(v_dev), m, n, offset,
                                                   group_size, kv_head_num, head_dim, dt, p(clock_probe_dev),
                                                   stream), "hip_flash_attn_gqa_clocked_layer")


def probe_mfma_ceiling(mix, target_ms=60.0):
    """Sustained bf16 MFMA TFLOP/s on N(0,1) operands: mix 0 = MFMAs alone, mix 1 = with the LDS reads and
    vector instructions of an attention inner loop beside them."""
    t = ctypes.c_double(0.0)
    _check(lib.llmhip_bench_mfma_ceiling(mix, float(target_ms), ctypes.byref(t)), "probe_mfma_ceiling")
    return t.value


def probe_stream_read(a, b, sink, variant, stream=None):
    """Enqueues a plain streaming read of the two equally sized device tensors a and b (what a kernel that
    only reads gets from the memory system)."""
    nbytes = a.numel() * a.element_size()
    if b.numel() * b.element_size() != nbytes:
        raise ValueError("probe_stream_read: a and b must have the same size")
    _check(lib.llmhip_bench_stream_read(ops._ptr(a), ops._ptr(b), nbytes, ops._ptr(sink),
                                        sink.numel() * sink.element_size(), variant, stream),
           "probe_stream_read")
