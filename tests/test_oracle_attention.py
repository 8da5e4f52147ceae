"""Pins the oracle's attention: textbook SDPA (library routine), float64 brute
force on tiny inputs, and invariants that a dropped term, a wrong mask bound or
a transposed operand would break."""
import numpy as np
import pytest
import torch

from helpers import TOL, normal_bits, ulp
from oracle import oracle as orc

F16, BF16 = orc.DT_FLOAT16, orc.DT_BFLOAT16


def _sdpa(q, k, v, n, offset, dt, dtype=torch.float64):
    """torch SDPA with an explicit boolean mask col <= row + offset and kv heads
    expanded with repeat_interleave (the HF repeat_kv convention)."""
    qf = torch.from_numpy(orc.widen(q, dt)).to(dtype)
    kf = torch.from_numpy(orc.widen(k[:n], dt)).to(dtype)
    vf = torch.from_numpy(orc.widen(v[:n], dt)).to(dtype)
    m, H, _ = qf.shape
    g = H // kf.shape[1]
    kf = kf.repeat_interleave(g, dim=1)
    vf = vf.repeat_interleave(g, dim=1)
    rows = torch.arange(m)[:, None]
    cols = torch.arange(n)[None, :]
    mask = cols <= rows + offset
    o = torch.nn.functional.scaled_dot_product_attention(
        qf.permute(1, 0, 2)[None], kf.permute(1, 0, 2)[None], vf.permute(1, 0, 2)[None],
        attn_mask=mask[None, None])
    return o[0].permute(1, 0, 2).numpy()


CASES = [(4, 4, 0, 2, 2), (3, 7, 4, 4, 2), (1, 33, 32, 6, 1), (9, 20, 11, 6, 3), (40, 40, 0, 4, 1)]


@pytest.mark.parametrize("dt", [F16, BF16])
@pytest.mark.parametrize("m,n,offset,H,Hkv", CASES)
def test_f32_oracle_equals_sdpa(dt, m, n, offset, H, Hkv):
    q = normal_bits(1, (m, H, 128), dt)
    k = normal_bits(2, (n + 3, Hkv, 128), dt)   # 3 rows past n must not be read
    v = normal_bits(3, (n + 3, Hkv, 128), dt)
    k[n:] = 0x7FFF
    v[n:] = 0x7FFF
    got = orc.attention_f32(q, k, v, n, offset, dt)
    want = _sdpa(q, k, v, n, offset, dt)
    assert np.abs(got - want).max() < 2e-5


@pytest.mark.parametrize("dt", [F16, BF16])
@pytest.mark.parametrize("m,n,offset,H,Hkv", CASES)
def test_layer_oracle_close_to_f32_oracle(dt, m, n, offset, H, Hkv):
    """How far apart the reference's two arithmetics are (layer path with storage
    rounding of scores, probabilities and output, src/llama2_layer_cpu.cpp:175-296,
    vs the fp32 test golden, tests/flash_attn_test.cpp:106-192).  fp16: half an
    output step plus less than half the 2e-3 bar.  bf16 (no reference code; the
    same chain with bf16 casts): probabilities rounded to 8 bits move rows that
    see only a few keys by up to ~1e-2 on their own, so the two differ by more
    than the bf16 bar; the fp32 golden is therefore the primary oracle and the
    layer-style one is compared with a one-step allowance."""
    q = normal_bits(4, (m, H, 128), dt)
    k = normal_bits(5, (n, Hkv, 128), dt)
    v = normal_bits(6, (n, Hkv, 128), dt)
    a = orc.attention_f32(q, k, v, n, offset, dt)
    b = orc.widen(orc.attention_layer(q, k, v, n, offset, dt), dt)
    slack = TOL[dt] / 2 if dt == F16 else 2 * TOL[dt]
    assert np.all(np.abs(a - b) <= slack + ulp(a, dt) / 2)


def test_brute_force_float64_tiny():
    rng = np.random.default_rng(9)
    for (m, n, offset, H, Hkv) in [(2, 3, 1, 2, 1), (5, 8, 3, 4, 2), (8, 8, 0, 1, 1)]:
        q = normal_bits(rng.integers(1 << 30), (m, H, 128), F16)
        k = normal_bits(rng.integers(1 << 30), (n, Hkv, 128), F16)
        v = normal_bits(rng.integers(1 << 30), (n, Hkv, 128), F16)
        qf, kf, vf = (orc.widen(a, F16).astype(np.float64) for a in (q, k, v))
        want = np.zeros((m, H, 128))
        g = H // Hkv
        for r in range(m):
            for h in range(H):
                sc = [qf[r, h] @ kf[c, h // g] / np.sqrt(128.0) if c <= r + offset else -np.inf for c in range(n)]
                e = np.exp(np.array(sc) - max(sc))
                p = e / e.sum()
                for c in range(n):
                    want[r, h] += p[c] * vf[c, h // g]
        assert np.abs(orc.attention_f32(q, k, v, n, offset, F16) - want).max() < 2e-5


def test_constant_v_gives_constant_output():
    """Rows of P sum to one."""
    q = normal_bits(21, (6, 4, 128), F16)
    k = normal_bits(22, (10, 2, 128), F16)
    v = np.full((10, 2, 128), orc.round_to(np.array([0.375], dtype=np.float32), F16)[0], dtype=np.uint16)
    out = orc.attention_f32(q, k, v, 10, 4, F16)
    assert np.abs(out - 0.375).max() < 1e-6


def test_single_key_and_first_causal_row_return_v0():
    q = normal_bits(23, (3, 4, 128), BF16)
    k = normal_bits(24, (5, 2, 128), BF16)
    v = normal_bits(25, (5, 2, 128), BF16)
    vf = orc.widen(v, BF16)
    one = orc.attention_f32(q, k, v, 1, 0, BF16)
    for h in range(4):
        assert np.array_equal(one[:, h], np.broadcast_to(vf[0, h // 2], (3, 128)))
    causal = orc.attention_f32(q, k, v, 5, 0, BF16)
    for h in range(4):
        assert np.array_equal(causal[0, h], vf[0, h // 2])


def test_mask_bound_is_col_greater_than_row_plus_offset():
    """Changing a key at column row+offset+1 must not change that row, changing the
    key at column row+offset must (src/llama2_layer_cpu.cpp:687-701)."""
    m, n, offset = 4, 9, 3
    q = normal_bits(26, (m, 1, 128), F16)
    k = normal_bits(27, (n, 1, 128), F16)
    v = normal_bits(28, (n, 1, 128), F16)
    base = orc.attention_f32(q, k, v, n, offset, F16)
    for r in range(m):
        v2 = v.copy()
        v2[r + offset + 1] = normal_bits(99, (1, 128), F16)
        assert np.array_equal(orc.attention_f32(q, k, v2, n, offset, F16)[r], base[r])
        v3 = v.copy()
        v3[r + offset] = normal_bits(98, (1, 128), F16)
        assert not np.array_equal(orc.attention_f32(q, k, v3, n, offset, F16)[r], base[r])


def test_gqa_equals_mha_on_repeated_kv():
    """q head h reads kv head h // group_size: identical to MHA over K/V expanded
    with repeat_interleave.  (The mapping is the HF repeat_kv convention; no
    reference source or test shows it -- parity unpinned at that point.)"""
    for dt in (F16, BF16):
        q = normal_bits(31, (7, 6, 128), dt)
        k = normal_bits(32, (12, 2, 128), dt)
        v = normal_bits(33, (12, 2, 128), dt)
        a = orc.attention_layer(q, k, v, 12, 5, dt)
        b = orc.attention_layer(q, np.repeat(k, 3, axis=1), np.repeat(v, 3, axis=1), 12, 5, dt)
        assert np.array_equal(a, b)


def test_prefill_row_equals_decode():
    q = normal_bits(34, (6, 4, 128), BF16)
    k = normal_bits(35, (10, 2, 128), BF16)
    v = normal_bits(36, (10, 2, 128), BF16)
    full = orc.attention_layer(q, k, v, 10, 4, BF16)
    for r in range(6):
        dec = orc.attention_layer(q[r:r + 1], k, v, r + 5, r + 4, BF16)
        assert np.array_equal(dec[0], full[r])


def test_key_permutation_invariance_of_decode():
    q = normal_bits(37, (1, 4, 128), F16)
    k = normal_bits(38, (50, 4, 128), F16)
    v = normal_bits(39, (50, 4, 128), F16)
    perm = np.random.default_rng(3).permutation(50)
    a = orc.attention_f32(q, k, v, 50, 49, F16)
    b = orc.attention_f32(q, np.ascontiguousarray(k[perm]), np.ascontiguousarray(v[perm]), 50, 49, F16)
    assert np.abs(a - b).max() < 1e-5


def test_batch_entries_are_independent():
    q = normal_bits(40, (3, 1, 4, 128), BF16)
    k = normal_bits(41, (3, 20, 2, 128), BF16)
    v = normal_bits(42, (3, 20, 2, 128), BF16)
    base = orc.attention_layer(q, k, v, 17, 16, BF16, batch=True)
    k2 = k.copy()
    k2[1] = normal_bits(43, (20, 2, 128), BF16)
    pert = orc.attention_layer(q, k2, v, 17, 16, BF16, batch=True)
    assert np.array_equal(base[0], pert[0]) and np.array_equal(base[2], pert[2])
    assert not np.array_equal(base[1], pert[1])
    for b in range(3):
        single = orc.attention_layer(q[b], k[b], v[b], 17, 16, BF16)
        assert np.array_equal(single, base[b])


def test_all_close_rule():
    """An element fails only if BOTH bounds are exceeded (tests/npu_op_test_util.cpp:41)."""
    a = np.array([1.0, 100.0, 1e-6, 1.0], dtype=np.float32)
    b = np.array([1.0005, 100.05, 5e-4, 1.01], dtype=np.float32)
    bad, mx = orc.all_close(a, b)
    assert bad == 1            # only the last: abs 0.01 > 1e-3 and rel 0.0099 > 1e-3
    assert abs(mx - 0.05) < 1e-3
