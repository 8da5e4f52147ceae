"""GPU parity of the projections either side of the attention block (through the C ABI):
hipBLASLt GEMM with fp32 bias epilogue and the residual add, against the oracle's
restatement of tests/gemm_test.cpp:138-149."""
import numpy as np
import pytest

from helpers import DT_BFLOAT16, DT_FLOAT16, dev_empty, f32_dev, normal_bits, to_dev, to_host, ulp
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def _ops():
    import llm_simple_amd.ops as ops
    return ops



# (m, n, k, bias): Qwen2.5-7B q/k/o projections (hidden 3584, kv dim 512), Qwen2.5-1.5B q (1536),
# and small ragged m
CASES = [
    (256, 3584, 3584, True),
    (256, 512, 3584, True),
    (256, 3584, 3584, False),
    (1, 3584, 3584, True),
    (17, 512, 3584, True),
    (5, 1536, 1536, True),
    (33, 48, 272, False),
]


@pytest.mark.parametrize("dt", [DT_FLOAT16, DT_BFLOAT16])
@pytest.mark.parametrize("m,n,k,bias", CASES)
def test_matmul_bias_vs_oracle(dt, m, n, k, bias):
    ops = _ops()
    x = normal_bits(100 + m, (m, k), dt)
    # weights of realistic scale: outputs stay O(1) like a trained projection
    w = orc.round_to(orc.widen(normal_bits(200 + n, (n, k), dt), dt) / np.sqrt(k), dt)
    b = np.random.default_rng(300 + n).standard_normal(n).astype(np.float32) if bias else None
    d_out = dev_empty((m, n))
    if bias:
        ops.hip_matmul_bias_layer(d_out, to_dev(x), to_dev(w), f32_dev(b), m, n, k, dt)
    else:
        ops.hip_matmul_layer(d_out, to_dev(x), to_dev(w), m, n, k, dt)
    got = orc.widen(to_host(d_out), dt)
    ref = orc.widen(orc.matmul_bias(x, w, b, dt), dt)
    # the reference's own rule for this operator: tests/gemm_test.cpp:163, all_close(0.01, 0.01)
    bad, mx = orc.all_close(got, ref, 0.01, 0.01)
    assert bad == 0, f"{bad} elements outside the reference rule, max abs {mx}"
    # and the sharper statement: both are one rounding of an fp32 sum whose order differs, so they
    # agree to one step of the storage type (or 1e-3 where the sum cancels)
    d = np.abs(got - ref)
    assert (d <= np.maximum(1.01 * ulp(ref, dt), 1e-3)).all(), f"worst {d.max()}"


@pytest.mark.parametrize("dt", [DT_FLOAT16, DT_BFLOAT16])
@pytest.mark.parametrize("total", [8, 1000, 256 * 3584, 256 * 3584 + 3])
def test_add_bit_exact(dt, total):
    ops = _ops()
    a = normal_bits(11, (total,), dt)
    b = normal_bits(12, (total,), dt)
    d_out = dev_empty((total,))
    ops.hip_add_layer(d_out, to_dev(a), to_dev(b), total, dt)
    assert np.array_equal(to_host(d_out), orc.add(a, b, dt))


def test_matmul_rejects_bad_arguments():
    ops = _ops()
    x = to_dev(normal_bits(1, (4, 32), DT_BFLOAT16))
    w = to_dev(normal_bits(2, (16, 32), DT_BFLOAT16))
    out = dev_empty((4, 16))
    with pytest.raises(ops.LlmHipError):
        ops.hip_matmul_layer(out, x, w, 4, 15, 32, DT_BFLOAT16)   # n not a multiple of 16
    with pytest.raises(ops.LlmHipError):
        ops.hip_matmul_layer(out, x, w, 4, 16, 32, 7)             # unknown dtype
    with pytest.raises(ops.LlmHipError):
        ops.hip_matmul_layer(out, x, w, 0, 16, 32, DT_BFLOAT16)   # m < 1


def test_release_then_reuse():
    """llmhip_release_internal_workspace() drops the hipBLASLt handle, plans and workspace (and the
    decode scratch); the next call builds them again."""
    ops = _ops()
    dt, m, n, k = DT_BFLOAT16, 8, 64, 128
    x = normal_bits(21, (m, k), dt)
    w = orc.round_to(orc.widen(normal_bits(22, (n, k), dt), dt) / np.sqrt(k), dt)
    ref = orc.widen(orc.matmul_bias(x, w, None, dt), dt)
    for _ in range(2):
        d_out = dev_empty((m, n))
        ops.hip_matmul_layer(d_out, to_dev(x), to_dev(w), m, n, k, dt)
        got = orc.widen(to_host(d_out), dt)
        assert (np.abs(got - ref) <= np.maximum(1.01 * ulp(ref, dt), 1e-3)).all()
        assert ops.lib.llmhip_device_sync() == 0
        assert ops.lib.llmhip_release_internal_workspace() == 0
