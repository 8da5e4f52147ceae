"""Pins of the oracle's projection GEMM (tests/gemm_test.cpp:138-149 restated) and residual add."""
import numpy as np
import pytest

from helpers import DT_BFLOAT16, DT_FLOAT16, normal_bits, ulp
from oracle import oracle as orc


@pytest.mark.parametrize("dt", [DT_FLOAT16, DT_BFLOAT16])
@pytest.mark.parametrize("m,n,k,bias", [(5, 32, 64, True), (33, 48, 272, False), (1, 16, 3584, True)])
def test_matmul_bias_vs_float64(dt, m, n, k, bias):
    x = normal_bits(1, (m, k), dt)
    w = normal_bits(2, (n, k), dt)
    b = np.random.default_rng(3).standard_normal(n).astype(np.float32) if bias else None
    got = orc.widen(orc.matmul_bias(x, w, b, dt), dt)
    ref = orc.widen(x, dt).astype(np.float64) @ orc.widen(w, dt).astype(np.float64).T
    if bias:
        ref = ref + b.astype(np.float64)
    # fp32 accumulation error (<= k * 2^-24 * sum|terms|) is far below one step of the storage type
    step = ulp(ref.astype(np.float32), dt)
    assert (np.abs(got - ref) <= 0.51 * step + 1e-6 * np.abs(ref) + k * 2.0 ** -22).all()


@pytest.mark.parametrize("dt", [DT_FLOAT16, DT_BFLOAT16])
def test_matmul_identity_zero_and_permutation(dt):
    k = n = 64
    x = normal_bits(4, (7, k), dt)
    eye = orc.round_to(np.eye(n, dtype=np.float32), dt)
    assert np.array_equal(orc.matmul_bias(x, eye, None, dt), x)            # x . I == x, exactly
    b = np.linspace(-3, 3, n).astype(np.float32)
    zero = np.zeros_like(x)
    w = normal_bits(5, (n, k), dt)
    assert np.array_equal(orc.matmul_bias(zero, w, b, dt), np.tile(orc.round_to(b, dt), (7, 1)))
    # a transposed weight (w[k][n] instead of w[n][k]) or a swapped operand would break this:
    perm = np.random.default_rng(6).permutation(n)
    rows = np.random.default_rng(7).permutation(7)
    full = orc.matmul_bias(x, w, b, dt)
    assert np.array_equal(orc.matmul_bias(x[rows], w[perm], b[perm], dt), full[rows][:, perm])


@pytest.mark.parametrize("dt", [DT_FLOAT16, DT_BFLOAT16])
def test_add_vs_numpy(dt):
    a = normal_bits(8, (1000,), dt)
    b = normal_bits(9, (1000,), dt)
    ref = orc.round_to(orc.widen(a, dt) + orc.widen(b, dt), dt)
    assert np.array_equal(orc.add(a, b, dt), ref)
