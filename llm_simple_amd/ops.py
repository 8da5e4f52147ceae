"""ctypes binding of libllmhip.so.

Function names and argument order follow the reference's operator header
(prebuild/npu_ops.h:6-18, :39-47) with the ``npu_`` prefix replaced by
``hip_``; device buffers are passed as raw addresses (``tensor.data_ptr()`` of
a torch tensor on the GPU, or any other device pointer) and the stream as a
``hipStream_t`` address (0 = default stream).  Every call is asynchronous on
its stream and raises :class:`LlmHipError` on a non-zero status.
"""
import ctypes
import math
import os

import numpy as np

DT_FLOAT16 = 4   # prebuild/defs.hpp:13
DT_BFLOAT16 = 5  # prebuild/defs.hpp:14

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libllmhip.so")

# Every symbol include/llmhip.h declares: (name, restype, argtypes)
_vp, _i, _i64, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t
SYMBOLS = {
    "llmhip_flash_attn": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "llmhip_flash_attn_gqa": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "llmhip_flash_attn_scratch_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "llmhip_flash_attn_opt_prefill": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "llmhip_flash_decode_gqa": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _i64, _i, _i, _i, _i, _i, _vp]),
    "llmhip_flash_decode_gqa_static": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i64, _i, _i, _i, _i, _i, _vp]),
    "llmhip_flash_decode_static_scratch_bytes": (_sz, []),
    "llmhip_decode_step_gqa": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "llmhip_flash_decode_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "llmhip_flash_decode_default_splits": (_i, [_i, _i, _i]),
    "llmhip_rope": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "llmhip_rope_single": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "llmhip_rope_kv_append": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "llmhip_matmul": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "llmhip_matmul_bias": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "llmhip_add": (_i, [_vp, _vp, _vp, ctypes.c_longlong, _i, _vp]),
    "llmhip_device_count": (_i, []),
    "llmhip_device_props": (_i, [_i, ctypes.POINTER(_i), ctypes.POINTER(_i), ctypes.POINTER(_sz)]),
    "llmhip_set_device": (_i, [_i]),
    "llmhip_malloc": (_i, [ctypes.POINTER(_vp), _sz]),
    "llmhip_free": (_i, [_vp]),
    "llmhip_memcpy_h2d": (_i, [_vp, _vp, _sz]),
    "llmhip_memcpy_d2h": (_i, [_vp, _vp, _sz]),
    "llmhip_memcpy_d2d_async": (_i, [_vp, _vp, _sz, _vp]),
    "llmhip_memset_async": (_i, [_vp, _i, _sz, _vp]),
    "llmhip_stream_create": (_i, [ctypes.POINTER(_vp)]),
    "llmhip_stream_destroy": (_i, [_vp]),
    "llmhip_stream_sync": (_i, [_vp]),
    "llmhip_device_sync": (_i, []),
    "llmhip_event_create": (_i, [ctypes.POINTER(_vp)]),
    "llmhip_event_destroy": (_i, [_vp]),
    "llmhip_event_record": (_i, [_vp, _vp]),
    "llmhip_event_sync": (_i, [_vp]),
    "llmhip_event_query": (_i, [_vp]),
    "llmhip_event_elapsed_ms": (_i, [ctypes.POINTER(ctypes.c_float), _vp, _vp]),
    "llmhip_error_string": (ctypes.c_char_p, [_i]),
    "llmhip_release_internal_workspace": (_i, []),
}


class LlmHipError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        msg = lib.llmhip_error_string(status)
        super().__init__(f"{where}: status {status} ({msg.decode() if msg else '?'})")


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C llm_simple_amd/csrc` "
            "(or __graft_entry__.build()); there is no CPU fallback")
    handle = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(handle, name)
        fn.restype = res
        fn.argtypes = args
    return handle


lib = _load()


def _check(status, where):
    if status != 0:
        raise LlmHipError(status, where)


def _ptr(x):
    """Device address of a torch tensor, or an int address passed through."""
    if x is None:
        return None
    if isinstance(x, int):
        return x
    return x.data_ptr()


def hip_flash_attn_layer(output_dev, q_dev, k_dev, v_dev, m, n, offset, head_num, head_dim, dt,
                         stream=0):
    """npu_flash_attn_layer (prebuild/npu_ops.h:6-8)."""
    _check(lib.llmhip_flash_attn(_ptr(output_dev), _ptr(q_dev), _ptr(k_dev), _ptr(v_dev), m, n,
                                 offset, head_num, head_dim, dt, stream), "hip_flash_attn_layer")


def hip_flash_attn_gqa_layer(output_dev, q_dev, k_dev, v_dev, m, n, offset, group_size,
                             kv_head_num, head_dim, dt, stream=0):
    """npu_flash_attn_gqa_layer (prebuild/npu_ops.h:10-13)."""
    _check(lib.llmhip_flash_attn_gqa(_ptr(output_dev), _ptr(q_dev), _ptr(k_dev), _ptr(v_dev), m,
                                     n, offset, group_size, kv_head_num, head_dim, dt, stream),
           "hip_flash_attn_gqa_layer")


def hip_flash_attn_opt_prefill_layer(output_dev, q_dev, k_dev, v_dev, m, n, offset, head_num,
                                     head_dim, dt, stream=0):
    """npu_flash_attn_opt_prefill_layer (prebuild/npu_ops.h:15-18)."""
    _check(lib.llmhip_flash_attn_opt_prefill(_ptr(output_dev), _ptr(q_dev), _ptr(k_dev),
                                             _ptr(v_dev), m, n, offset, head_num, head_dim, dt,
                                             stream), "hip_flash_attn_opt_prefill_layer")


def hip_flash_decode_gqa_layer(output_dev, q_dev, k_cache_dev, v_cache_dev, workspace_dev,
                               workspace_bytes, batch, n, kv_seq_stride, group_size, kv_head_num,
                               head_dim, num_splits, dt, stream=0):
    """Batched split-KV decode (no counterpart in the reference header: decode there
    is npu_flash_attn_gqa_layer with m = 1, src/llama2_layer_npu.cpp:866-869)."""
    _check(lib.llmhip_flash_decode_gqa(_ptr(output_dev), _ptr(q_dev), _ptr(k_cache_dev),
                                       _ptr(v_cache_dev), _ptr(workspace_dev), workspace_bytes,
                                       batch, n, kv_seq_stride, group_size, kv_head_num, head_dim,
                                       num_splits, dt, stream), "hip_flash_decode_gqa_layer")


def hip_flash_decode_gqa_static_layer(output_dev, q_dev, k_cache_dev, v_cache_dev, batch, n,
                                      kv_seq_stride, group_size, kv_head_num, head_dim, num_splits, dt,
                                      stream=0):
    """hip_flash_decode_gqa_layer without a workspace: the partials live in a fixed 4 MiB array
    inside the library and the call allocates nothing."""
    _check(lib.llmhip_flash_decode_gqa_static(_ptr(output_dev), _ptr(q_dev), _ptr(k_cache_dev),
                                              _ptr(v_cache_dev), batch, n, kv_seq_stride, group_size,
                                              kv_head_num, head_dim, num_splits, dt, stream),
           "hip_flash_decode_gqa_static_layer")


def hip_decode_step_gqa_layer(output_dev, k_cache_dev, v_cache_dev, freqs_cis_dev, input_q_dev, input_k_dev,
                              input_v_dev, pos, group_size, kv_head_num, head_dim, is_neox_style, dt, stream=0):
    """One decode step in one pass over the cache: rope(q), rope(k) -> k_cache[pos], v -> v_cache[pos] and
    attention over rows [0, pos], fused into the decode kernel (src/llama2_layer_npu.cpp:790-869 does it
    with four calls)."""
    _check(lib.llmhip_decode_step_gqa(_ptr(output_dev), _ptr(k_cache_dev), _ptr(v_cache_dev),
                                      _ptr(freqs_cis_dev), _ptr(input_q_dev), _ptr(input_k_dev),
                                      _ptr(input_v_dev), pos, group_size, kv_head_num, head_dim,
                                      int(bool(is_neox_style)), dt, stream), "hip_decode_step_gqa_layer")


def flash_decode_workspace_bytes(batch, group_size, kv_head_num, head_dim, num_splits):
    return lib.llmhip_flash_decode_workspace_bytes(batch, group_size, kv_head_num, head_dim,
                                                   num_splits)


def flash_decode_default_splits(batch, n, kv_head_num):
    return lib.llmhip_flash_decode_default_splits(batch, n, kv_head_num)


def hip_matmul_layer(output_dev, lhs_dev, weight_dev, m, n, k, dt, stream=0):
    """npu_matmul_nz_layer (prebuild/npu_ops.h:87-88) with the weight as W[n][k] row-major."""
    _check(lib.llmhip_matmul(_ptr(output_dev), _ptr(lhs_dev), _ptr(weight_dev), m, n, k, dt, stream),
           "hip_matmul_layer")


def hip_matmul_bias_layer(output_dev, lhs_dev, weight_dev, bias_dev, m, n, k, dt, stream=0):
    """npu_matmul_bias_nz_layer (prebuild/npu_ops.h:90-92): fp32 bias added before the rounding."""
    _check(lib.llmhip_matmul_bias(_ptr(output_dev), _ptr(lhs_dev), _ptr(weight_dev), _ptr(bias_dev),
                                  m, n, k, dt, stream), "hip_matmul_bias_layer")


def hip_add_layer(output_dev, lhs_dev, rhs_dev, total_size, dt, stream=0):
    """npu_add_layer (prebuild/npu_ops.h:81-82)."""
    _check(lib.llmhip_add(_ptr(output_dev), _ptr(lhs_dev), _ptr(rhs_dev), total_size, dt, stream),
           "hip_add_layer")


def hip_rope_layer(output_q_dev, output_k_dev, freqs_cis_dev, input_q_dev, input_k_dev, start_pos,
                   cur_size, n_heads, hidden_dim, is_neox_style, dt, stream=0):
    """npu_rope_layer (prebuild/npu_ops.h:39-42)."""
    _check(lib.llmhip_rope(_ptr(output_q_dev), _ptr(output_k_dev), _ptr(freqs_cis_dev),
                           _ptr(input_q_dev), _ptr(input_k_dev), start_pos, cur_size, n_heads,
                           hidden_dim, int(bool(is_neox_style)), dt, stream), "hip_rope_layer")


def hip_rope_single_layer(output_x_dev, freqs_cis_dev, input_x_dev, start_pos, cur_size, n_heads,
                          hidden_dim, is_neox_style, dt, stream=0):
    """npu_rope_single_layer (prebuild/npu_ops.h:44-47)."""
    _check(lib.llmhip_rope_single(_ptr(output_x_dev), _ptr(freqs_cis_dev), _ptr(input_x_dev),
                                  start_pos, cur_size, n_heads, hidden_dim,
                                  int(bool(is_neox_style)), dt, stream), "hip_rope_single_layer")


def hip_rope_kv_append_layer(output_q_dev, k_cache_dev, v_cache_dev, freqs_cis_dev, input_q_dev,
                             input_k_dev, input_v_dev, start_pos, cur_size, n_heads, n_kv_heads,
                             head_dim, is_neox_style, dt, stream=0):
    """rope(Q), rope(K) -> k_cache[start_pos:], V -> v_cache[start_pos:] in one launch
    (src/llama2_layer_npu.cpp:790-798 + :830-844)."""
    _check(lib.llmhip_rope_kv_append(_ptr(output_q_dev), _ptr(k_cache_dev), _ptr(v_cache_dev),
                                     _ptr(freqs_cis_dev), _ptr(input_q_dev), _ptr(input_k_dev),
                                     _ptr(input_v_dev), start_pos, cur_size, n_heads, n_kv_heads,
                                     head_dim, int(bool(is_neox_style)), dt, stream),
           "hip_rope_kv_append_layer")


def device_props(device=0):
    """(compute units, maximum shader clock in MHz, memory bytes) of a device."""
    cus, khz, mem = _i(0), _i(0), _sz(0)
    _check(lib.llmhip_device_props(device, ctypes.byref(cus), ctypes.byref(khz), ctypes.byref(mem)),
           "device_props")
    return cus.value, khz.value / 1e3, mem.value


def _bf16_round_trip(x):
    """fp32 array -> nearest-even bf16 -> fp32, on the bit pattern."""
    u = x.astype(np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def init_freq_cis(head_dim, max_seq_len, theta=10000.0, dt=DT_FLOAT16):
    """Host-side rotary table, ModelBase::InitFreqCIS (src/model_base.cpp:27-83):
    inv_freq through a double pow then cast to float, angle = float(t) * inv_freq
    in fp32, (cos, sin) interleaved as [max_seq_len][head_dim/2][2] fp32, and for
    bf16 models every entry rounded to bf16 and widened back (:59-66)."""
    freq_len = head_dim // 2
    i2 = np.arange(freq_len, dtype=np.float64) * 2.0
    inv = (np.float32(1.0) / np.power(np.float64(np.float32(theta)), i2 / float(head_dim))).astype(np.float32)
    t = np.arange(max_seq_len, dtype=np.float32)
    ang = (t[:, None] * inv[None, :]).astype(np.float32)
    out = np.empty((max_seq_len, freq_len, 2), dtype=np.float32)
    # libm cosf/sinf through the scalar loop would be exact to the reference's
    # std::cos(float); numpy's float32 cos/sin are within 1 ulp of it
    out[..., 0] = np.cos(ang)
    out[..., 1] = np.sin(ang)
    if dt == DT_BFLOAT16:
        out = _bf16_round_trip(out.reshape(-1)).reshape(max_seq_len, freq_len, 2)
    return out


def attention_scale(head_dim):
    """1/sqrtf(head_dim), src/llama2_layer_cpu.cpp:177."""
    return 1.0 / math.sqrt(float(head_dim))
