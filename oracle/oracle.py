"""ctypes front end of oracle/liboracle.so -- TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may
import this module.  Arrays of 16-bit storage values travel as numpy uint16.
"""
import ctypes
import os
import subprocess

import numpy as np

DT_FLOAT16 = 4
DT_BFLOAT16 = 5

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")


def build(force=False):
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"])
    return _SO


def _load():
    build()
    h = ctypes.CDLL(_SO)
    vp, i, i64, f = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
    h.orc_f32_to_bf16.restype = ctypes.c_uint16
    h.orc_f32_to_bf16.argtypes = [ctypes.c_uint32]
    h.orc_bf16_to_f32.restype = f
    h.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
    h.orc_f32_to_f16.restype = ctypes.c_uint16
    h.orc_f32_to_f16.argtypes = [f]
    h.orc_f16_to_f32.restype = f
    h.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
    h.orc_round_array.argtypes = [vp, vp, i64, i]
    h.orc_widen_array.argtypes = [vp, vp, i64, i]
    h.orc_init_freq_cis.argtypes = [vp, i, i, f, i, i]
    h.orc_rope.argtypes = [vp, vp, vp, i, i, i, i, i, i]
    h.orc_kv_append.argtypes = [vp, vp, i, i, i]
    h.orc_attention_layer.argtypes = [vp, vp, vp, vp, i, i, i, i, i, i, i, i64, i, i]
    h.orc_attention_f32.argtypes = [vp, vp, vp, vp, i, i, i, i, i, i, i, i64, i, i]
    h.orc_matmul_bias.argtypes = [vp, vp, vp, vp, i, i, i, i, i]
    h.orc_add.argtypes = [vp, vp, vp, i64, i]
    h.orc_all_close.restype = i64
    h.orc_all_close.argtypes = [vp, vp, i64, f, f, ctypes.POINTER(f)]
    h.orc_max_threads.restype = i
    return h


_h = _load()


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def round_to(x, dt):
    """fp32 array -> storage bits (uint16), round to nearest even."""
    x = _c(x, np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    _h.orc_round_array(_p(out), _p(x), x.size, dt)
    return out


def widen(bits, dt):
    bits = _c(bits, np.uint16)
    out = np.empty(bits.shape, dtype=np.float32)
    _h.orc_widen_array(_p(out), _p(bits), bits.size, dt)
    return out


def f32_to_bf16_scalar(bits):
    return int(_h.orc_f32_to_bf16(ctypes.c_uint32(bits)))


def f32_to_f16_scalar(x):
    return int(_h.orc_f32_to_f16(ctypes.c_float(x)))


def init_freq_cis(head_dim, max_seq_len, theta, dt, use_powf=False):
    out = np.empty((max_seq_len, head_dim // 2, 2), dtype=np.float32)
    _h.orc_init_freq_cis(_p(out), head_dim, max_seq_len, ctypes.c_float(theta), dt, int(use_powf))
    return out


def rope(x_bits, freq_cis, start_pos, is_neox, dt):
    """x_bits: uint16 [cur_size][n_heads][head_dim] -> rotated uint16, same shape."""
    x_bits = _c(x_bits, np.uint16)
    freq_cis = _c(freq_cis, np.float32)
    cur_size, n_heads, head_dim = x_bits.shape
    assert start_pos + cur_size <= freq_cis.shape[0]
    out = np.empty_like(x_bits)
    _h.orc_rope(_p(out), _p(x_bits), _p(freq_cis), start_pos, cur_size, n_heads, head_dim,
                int(bool(is_neox)), dt)
    return out


def kv_append(cache_bits, src_bits, prev_pos):
    """In place: cache[prev_pos:prev_pos+cur_size] = src (both uint16, [rows][...])."""
    assert cache_bits.dtype == np.uint16 and cache_bits.flags.c_contiguous
    src_bits = _c(src_bits, np.uint16)
    cur_size = src_bits.shape[0]
    row_elems = int(np.prod(src_bits.shape[1:]))
    assert int(np.prod(cache_bits.shape[1:])) == row_elems
    assert prev_pos + cur_size <= cache_bits.shape[0]
    _h.orc_kv_append(_p(cache_bits), _p(src_bits), prev_pos, cur_size, row_elems)


def _attn_args(q, k, v, n, offset, batch):
    q = _c(q, np.uint16)
    k = _c(k, np.uint16)
    v = _c(v, np.uint16)
    if batch is None:
        assert q.ndim == 3 and k.ndim == 3
        b, (m, H, hd) = 1, q.shape
        stride, Hkv = k.shape[0], k.shape[1]
    else:
        assert q.ndim == 4 and k.ndim == 4
        b, m, H, hd = q.shape
        stride, Hkv = k.shape[1], k.shape[2]
    assert H % Hkv == 0 and k.shape == v.shape and n <= stride
    return q, k, v, b, m, H, Hkv, hd, stride


def attention_layer(q, k, v, n, offset, dt, batch=None, n_threads=0):
    """Layer-style attention (intermediate rounding to the storage type).
    q uint16 [m][H][hd] (or [B][m][H][hd] with batch=True), k/v uint16
    [rows][Hkv][hd] (or [B][rows][Hkv][hd]); rows [0,n) are read.
    Returns uint16 with q's shape."""
    q, k, v, b, m, H, Hkv, hd, stride = _attn_args(q, k, v, n, offset, batch)
    out = np.empty(q.shape, dtype=np.uint16)
    _h.orc_attention_layer(_p(out), _p(q), _p(k), _p(v), b, m, n, offset, H // Hkv, Hkv, hd,
                           stride, dt, n_threads)
    return out


def attention_f32(q, k, v, n, offset, dt, batch=None, n_threads=0):
    """fp32 end-to-end attention (the reference test golden); returns float32."""
    q, k, v, b, m, H, Hkv, hd, stride = _attn_args(q, k, v, n, offset, batch)
    out = np.empty(q.shape, dtype=np.float32)
    _h.orc_attention_f32(_p(out), _p(q), _p(k), _p(v), b, m, n, offset, H // Hkv, Hkv, hd,
                         stride, dt, n_threads)
    return out


def matmul_bias(lhs_bits, w_bits, bias, dt, n_threads=0):
    """round(lhs[m][k] . w[n][k]^T + bias[n]) -> bits [m][n]; bias fp32 or None."""
    lhs_bits = _c(lhs_bits, np.uint16)
    w_bits = _c(w_bits, np.uint16)
    m, k = lhs_bits.shape
    n, k2 = w_bits.shape
    assert k == k2
    out = np.empty((m, n), dtype=np.uint16)
    b = None if bias is None else _c(bias, np.float32)
    assert b is None or b.shape == (n,)
    _h.orc_matmul_bias(_p(out), _p(lhs_bits), _p(w_bits), None if b is None else _p(b), m, n, k, dt,
                       n_threads)
    return out


def add(lhs_bits, rhs_bits, dt):
    lhs_bits = _c(lhs_bits, np.uint16)
    rhs_bits = _c(rhs_bits, np.uint16)
    assert lhs_bits.shape == rhs_bits.shape
    out = np.empty(lhs_bits.shape, dtype=np.uint16)
    _h.orc_add(_p(out), _p(lhs_bits), _p(rhs_bits), lhs_bits.size, dt)
    return out


def all_close(a, b, abs_err=1e-3, rel_err=1e-3):
    """(failing element count, max abs error) under the reference's test rule."""
    a = _c(a, np.float32).reshape(-1)
    b = _c(b, np.float32).reshape(-1)
    mx = ctypes.c_float(0)
    bad = _h.orc_all_close(_p(a), _p(b), a.size, abs_err, rel_err, ctypes.byref(mx))
    return int(bad), float(mx.value)


def max_threads():
    return int(_h.orc_max_threads())
