"""Pins the oracle's RoPE and KV append by what the mathematics fixes."""
import numpy as np

from helpers import normal_bits
from oracle import oracle as orc

F16, BF16 = orc.DT_FLOAT16, orc.DT_BFLOAT16


def _complex_rope(x, tab, start, is_neox):
    """Brute force in float64: (a + ib)(cos + i sin) per pair."""
    s, h, d = x.shape
    out = np.empty_like(x, dtype=np.float64)
    for t in range(s):
        cs = tab[start + t].astype(np.float64)
        rot = cs[:, 0] + 1j * cs[:, 1]
        for j in range(h):
            row = x[t, j].astype(np.float64)
            if is_neox:
                z = (row[:64] + 1j * row[64:]) * rot
                out[t, j, :64], out[t, j, 64:] = z.real, z.imag
            else:
                z = (row[0::2] + 1j * row[1::2]) * rot
                out[t, j, 0::2], out[t, j, 1::2] = z.real, z.imag
    return out


def test_rope_equals_complex_multiplication():
    for dt, eps in ((F16, 2.0 ** -11), (BF16, 2.0 ** -8)):
        tab = orc.init_freq_cis(128, 300, 1e4, F16)
        x = normal_bits(11, (9, 3, 128), dt)
        xf = orc.widen(x, dt)
        for neox in (False, True):
            got = orc.widen(orc.rope(x, tab, 37, neox, dt), dt).astype(np.float64)
            want = _complex_rope(xf, tab, 37, neox)
            # one rounding to the storage type of a value of magnitude |want|
            assert np.all(np.abs(got - want) <= eps * np.abs(want) + 1e-6)


def test_rope_position_zero_is_identity():
    tab = orc.init_freq_cis(128, 4, 1e4, F16)
    for dt in (F16, BF16):
        x = normal_bits(12, (1, 5, 128), dt)
        for neox in (False, True):
            assert np.array_equal(orc.rope(x, tab, 0, neox, dt), x)


def test_rope_uses_start_pos_rows():
    """Row s of the input is rotated by table row start_pos + s (the device contract,
    tests/rope_single_layer_test.cpp:81-82), not by row s."""
    tab = orc.init_freq_cis(128, 64, 1e4, F16)
    x = normal_bits(13, (4, 2, 128), F16)
    whole = orc.rope(x, tab, 10, False, F16)
    for s in range(4):
        one = orc.rope(x[s:s + 1], tab, 10 + s, False, F16)
        assert np.array_equal(whole[s:s + 1], one)
    assert not np.array_equal(whole, orc.rope(x, tab, 0, False, F16))


def test_rope_preserves_pair_norm():
    tab = orc.init_freq_cis(128, 2048, 1e4, F16)
    x = normal_bits(14, (16, 4, 128), F16)
    xf = orc.widen(x, F16).astype(np.float64)
    y = orc.widen(orc.rope(x, tab, 1000, False, F16), F16).astype(np.float64)
    n_in = xf[..., 0::2] ** 2 + xf[..., 1::2] ** 2
    n_out = y[..., 0::2] ** 2 + y[..., 1::2] ** 2
    assert np.all(np.abs(n_in - n_out) <= 4e-3 * np.maximum(n_in, 1e-3))


def test_neox_is_interleaved_under_fixed_permutation():
    """neox on x == interleaved on x permuted by 2f -> f, 2f+1 -> f+64 (bit exact:
    the same fp32 operations on the same operands)."""
    tab = orc.init_freq_cis(128, 128, 1e6, BF16)
    for dt in (F16, BF16):
        x = normal_bits(15, (6, 3, 128), dt)
        perm = np.empty(128, dtype=np.int64)
        perm[0::2] = np.arange(64)
        perm[1::2] = np.arange(64) + 64
        inter = orc.rope(np.ascontiguousarray(x[..., perm]), tab, 5, False, dt)
        neox = orc.rope(x, tab, 5, True, dt)
        assert np.array_equal(neox[..., perm], inter)


def test_rope_composes_in_float64():
    """Rotation by p1 then p2 == rotation by p1 + p2 up to storage rounding."""
    tab = orc.init_freq_cis(128, 64, 1e4, F16)
    x = normal_bits(16, (1, 2, 128), F16)
    a = orc.rope(orc.rope(x, tab, 7, False, F16), tab, 9, False, F16)
    b = orc.rope(x, tab, 16, False, F16)
    assert np.abs(orc.widen(a, F16) - orc.widen(b, F16)).max() < 8e-3


def test_kv_append_canary():
    cache = np.full((32, 4, 128), 0xBEEF, dtype=np.uint16)
    src = normal_bits(17, (5, 4, 128), BF16)
    orc.kv_append(cache, src, 20)
    assert np.array_equal(cache[20:25], src)
    assert np.all(cache[:20] == 0xBEEF) and np.all(cache[25:] == 0xBEEF)
