"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle
on identical seeded inputs.  Bit-exact for RoPE and the KV append; max-abs
<= 2e-3 (fp16) / 1e-2 (bf16) on the attention output."""
import numpy as np
import pytest

from helpers import (DT_BFLOAT16, DT_FLOAT16, DT_NAME, TOL, check_attention, dev_empty, f32_dev,
                     normal_bits, to_dev, to_host)
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def _ops():
    import llm_simple_amd.ops as ops
    return ops


# ---------------------------------------------------------------- RoPE

@pytest.mark.parametrize("dt", [DT_FLOAT16, DT_BFLOAT16])
@pytest.mark.parametrize("is_neox", [False, True])
@pytest.mark.parametrize("cur_size,start_pos,n_heads", [(1, 0, 1), (1, 511, 32), (7, 3, 12), (256, 0, 28), (33, 2015, 4)])
def test_rope_single_bit_exact(dt, is_neox, cur_size, start_pos, n_heads):
    ops = _ops()
    theta = 10000.0 if dt == DT_FLOAT16 else 1e6
    table = orc.init_freq_cis(128, 2048, theta, dt)
    x = normal_bits(100 + cur_size + n_heads, (cur_size, n_heads, 128), dt)
    want = orc.rope(x, table, start_pos, is_neox, dt)
    d_out = dev_empty(x.shape)
    ops.hip_rope_single_layer(d_out, f32_dev(table), to_dev(x), start_pos, cur_size, n_heads,
                              n_heads * 128, is_neox, dt)
    got = to_host(d_out)
    assert np.array_equal(got, want), f"{np.count_nonzero(got != want)} elements differ"


@pytest.mark.parametrize("dt", [DT_FLOAT16, DT_BFLOAT16])
@pytest.mark.parametrize("is_neox", [False, True])
def test_rope_pair_bit_exact(dt, is_neox):
    ops = _ops()
    table = orc.init_freq_cis(128, 1024, 10000.0, dt)
    q = normal_bits(7, (19, 8, 128), dt)
    k = normal_bits(8, (19, 8, 128), dt)
    d_q, d_k = dev_empty(q.shape), dev_empty(k.shape)
    ops.hip_rope_layer(d_q, d_k, f32_dev(table), to_dev(q), to_dev(k), 100, 19, 8, 8 * 128,
                       is_neox, dt)
    assert np.array_equal(to_host(d_q), orc.rope(q, table, 100, is_neox, dt))
    assert np.array_equal(to_host(d_k), orc.rope(k, table, 100, is_neox, dt))


@pytest.mark.parametrize("dt,H,Hkv,theta", [(DT_FLOAT16, 32, 32, 1e4), (DT_BFLOAT16, 12, 2, 1e6), (DT_BFLOAT16, 28, 4, 1e6)])
@pytest.mark.parametrize("is_neox", [False, True])
@pytest.mark.parametrize("cur_size,start_pos", [(1, 511), (256, 0), (5, 250)])
def test_rope_kv_append_bit_exact(dt, H, Hkv, theta, is_neox, cur_size, start_pos):
    """Fused launch == unfused rope -> copy sequence of the oracle; rows outside
    [start_pos, start_pos+cur_size) of both caches keep their canary bytes."""
    ops = _ops()
    max_seq = 512
    table = orc.init_freq_cis(128, max_seq, theta, dt)
    q = normal_bits(1, (cur_size, H, 128), dt)
    k = normal_bits(2, (cur_size, Hkv, 128), dt)
    v = normal_bits(3, (cur_size, Hkv, 128), dt)
    canary_k = np.full((max_seq, Hkv, 128), 0xBEEF, dtype=np.uint16)
    canary_v = np.full((max_seq, Hkv, 128), 0xCAFE, dtype=np.uint16)
    want_k, want_v = canary_k.copy(), canary_v.copy()
    orc.kv_append(want_k, orc.rope(k, table, start_pos, is_neox, dt), start_pos)
    orc.kv_append(want_v, v, start_pos)
    want_q = orc.rope(q, table, start_pos, is_neox, dt)
    d_q, d_kc, d_vc = dev_empty(q.shape), to_dev(canary_k), to_dev(canary_v)
    ops.hip_rope_kv_append_layer(d_q, d_kc, d_vc, f32_dev(table), to_dev(q), to_dev(k), to_dev(v),
                                 start_pos, cur_size, H, Hkv, 128, is_neox, dt)
    assert np.array_equal(to_host(d_q), want_q)
    assert np.array_equal(to_host(d_kc), want_k)
    assert np.array_equal(to_host(d_vc), want_v)


# ---------------------------------------------------------------- attention

ATTN_CASES = [
    # (m, n, offset, H, Hkv)
    (4, 4, 0, 2, 2),
    (3, 7, 4, 4, 2),
    (1, 33, 32, 6, 1),
    (17, 17, 0, 3, 1),
    (64, 64, 0, 8, 8),
    (65, 129, 64, 8, 2),
    (128, 128, 0, 4, 4),
    (200, 333, 133, 14, 2),
    (256, 256, 0, 12, 2),
    (300, 300, 0, 28, 4),
    (77, 590, 513, 28, 4),
    (513, 513, 0, 5, 5),
    # n < m + offset: the cache length, not the causal bound, cuts the last rows
    (40, 50, 30, 4, 2),
    (300, 320, 100, 8, 2),
    (9, 10, 5, 2, 1),
]


@pytest.mark.parametrize("dt", [DT_FLOAT16, DT_BFLOAT16])
@pytest.mark.parametrize("m,n,offset,H,Hkv", ATTN_CASES)
def test_flash_attn_gqa_vs_oracle(dt, m, n, offset, H, Hkv):
    ops = _ops()
    seed = 1000 * m + n + H
    q = normal_bits(seed, (m, H, 128), dt)
    k = normal_bits(seed + 1, (n, Hkv, 128), dt)
    v = normal_bits(seed + 2, (n, Hkv, 128), dt)
    d_out = dev_empty(q.shape)
    ops.hip_flash_attn_gqa_layer(d_out, to_dev(q), to_dev(k), to_dev(v), m, n, offset, H // Hkv,
                                 Hkv, 128, dt)
    check_attention(to_host(d_out), q, k, v, n, offset, dt)


def _random_shapes():
    """Seeded shape sweep: every loop-exit case of the prefill kernels (1..11 key tiles per
    workgroup, ragged tails, offsets that put the diagonal anywhere in a tile), both the
    4-wave and the 8-wave kernel (the latter needs ceil(m/256)*H >= 384)."""
    rng = np.random.default_rng(20240607)
    shapes = []
    for i in range(36):
        big = i % 3 == 0
        m = int(rng.integers(17, 700))
        offset = int(rng.choice([0, 0, 1, 31, 63, 64, 65, int(rng.integers(0, 400))]))
        Hkv = int(rng.choice([1, 2, 4, 8]))
        g = int(rng.choice([1, 2, 5, 7]))
        if big:
            tiles = -(-m // 256)
            while tiles * Hkv * g < 384:
                Hkv *= 2
        shapes.append((m, m + offset, offset, Hkv * g, Hkv))
    return shapes


@pytest.mark.parametrize("idx,shape", list(enumerate(_random_shapes())))
def test_flash_attn_shape_sweep(idx, shape):
    ops = _ops()
    m, n, offset, H, Hkv = shape
    dt = DT_BFLOAT16 if idx % 2 else DT_FLOAT16
    q = normal_bits(7000 + idx, (m, H, 128), dt)
    k = normal_bits(7100 + idx, (n, Hkv, 128), dt)
    v = normal_bits(7200 + idx, (n, Hkv, 128), dt)
    d_out = dev_empty(q.shape)
    ops.hip_flash_attn_gqa_layer(d_out, to_dev(q), to_dev(k), to_dev(v), m, n, offset, H // Hkv,
                                 Hkv, 128, dt)
    check_attention(to_host(d_out), q, k, v, n, offset, dt)


@pytest.mark.parametrize("dt", [DT_FLOAT16, DT_BFLOAT16])
@pytest.mark.parametrize("H,Hkv", [(4, 2), (96, 8)])
def test_flash_attn_late_large_scores(dt, H, Hkv):
    """Scores that grow along the key axis: the reference maximum of the online softmax has to
    move many times, late in the key loop (the rescale path of the kernels), for the 4-wave
    (H=4) and the 8-wave (H=96, m=1024) kernel."""
    ops = _ops()
    m = n = 1024
    q = orc.widen(normal_bits(811, (m, H, 128), dt), dt)
    k = orc.widen(normal_bits(812, (n, Hkv, 128), dt), dt)
    v = normal_bits(813, (n, Hkv, 128), dt)
    ramp = (1.0 + 3.0 * np.arange(n, dtype=np.float32) / n)[:, None, None]
    q = orc.round_to(np.abs(q), dt)
    k = orc.round_to(np.abs(k) * ramp, dt)
    d_out = dev_empty(q.shape)
    ops.hip_flash_attn_gqa_layer(d_out, to_dev(q), to_dev(k), to_dev(v), m, n, 0, H // Hkv, Hkv, 128, dt)
    check_attention(to_host(d_out), q, k, v, n, 0, dt, layer_style=False)


def test_llama2_prefill_config_fp16():
    """Benchmark configuration 1: Llama2-7B prefill, fp16, H = Hkv = 32, m = n = 256, through the
    MHA entry point and the reference's own tolerance rule
    (tests/npu_op_test_util.cpp:33-48: abs 1e-3 AND rel 1e-3)."""
    ops = _ops()
    dt, m, H = DT_FLOAT16, 256, 32
    q = normal_bits(1001, (m, H, 128), dt)
    k = normal_bits(1002, (m, H, 128), dt)
    v = normal_bits(1003, (m, H, 128), dt)
    for fn in (ops.hip_flash_attn_layer, ops.hip_flash_attn_opt_prefill_layer):
        d_out = dev_empty(q.shape)
        fn(d_out, to_dev(q), to_dev(k), to_dev(v), m, m, 0, H, 128, dt)
        out = to_host(d_out)
        check_attention(out, q, k, v, m, 0, dt)
        bad, _ = orc.all_close(orc.widen(out, dt), orc.attention_f32(q, k, v, m, 0, dt))
        assert bad == 0


def test_llama2_prefill_then_decode_chain_fp16():
    """Benchmark configurations 1 and 2 through the whole path at full shape: Llama2-7B, fp16, H = Hkv = 32,
    theta 10000, interleaved RoPE (src/llama2_main.cpp:123-126).  Prefill: 256 tokens rotated, appended
    at rows 0..255, attended.  Decode: a cache of 511 rows, the new token rotated at position 511 and
    appended at row 511, attention m=1, n=512, offset=511.  Rotated Q and both caches bit-exact, the
    attention output against both oracles and the reference's all_close rule."""
    ops = _ops()
    dt, H, max_seq = DT_FLOAT16, 32, 512
    table = orc.init_freq_cis(128, max_seq, 10000.0, dt)
    d_table = f32_dev(table)
    # --- config 1
    m = 256
    q, k, v = (normal_bits(1001 + i, (m, H, 128), dt) for i in range(3))
    kc = np.full((max_seq, H, 128), 0x7FFF, dtype=np.uint16)  # NaN patterns: rows >= n must not be read
    vc = kc.copy()
    d_q, d_kc, d_vc, d_o = dev_empty(q.shape), to_dev(kc), to_dev(vc), dev_empty(q.shape)
    ops.hip_rope_kv_append_layer(d_q, d_kc, d_vc, d_table, to_dev(q), to_dev(k), to_dev(v), 0, m, H, H, 128,
                                 False, dt)
    ops.hip_flash_attn_layer(d_o, d_q, d_kc, d_vc, m, m, 0, H, 128, dt)
    q_r = orc.rope(q, table, 0, False, dt)
    orc.kv_append(kc, orc.rope(k, table, 0, False, dt), 0)
    orc.kv_append(vc, v, 0)
    assert np.array_equal(to_host(d_q), q_r)
    assert np.array_equal(to_host(d_kc), kc) and np.array_equal(to_host(d_vc), vc)
    out = to_host(d_o)
    check_attention(out, q_r, kc, vc, m, 0, dt)
    bad, _ = orc.all_close(orc.widen(out, dt), orc.attention_f32(q_r, kc, vc, m, 0, dt))
    assert bad == 0
    # --- config 2: rows 256..510 are "generated" tokens already in the cache
    kc[m:511] = normal_bits(1002, (511 - m, H, 128), dt)
    vc[m:511] = normal_bits(1012, (511 - m, H, 128), dt)
    d_kc, d_vc = to_dev(kc), to_dev(vc)
    q1, k1, v1 = (normal_bits(1020 + i, (1, H, 128), dt) for i in range(3))
    d_q1, d_o1 = dev_empty(q1.shape), dev_empty(q1.shape)
    ops.hip_rope_kv_append_layer(d_q1, d_kc, d_vc, d_table, to_dev(q1), to_dev(k1), to_dev(v1), 511, 1, H, H,
                                 128, False, dt)
    ops.hip_flash_attn_layer(d_o1, d_q1, d_kc, d_vc, 1, 512, 511, H, 128, dt)
    q1_r = orc.rope(q1, table, 511, False, dt)
    orc.kv_append(kc, orc.rope(k1, table, 511, False, dt), 511)
    orc.kv_append(vc, v1, 511)
    assert np.array_equal(to_host(d_q1), q1_r)
    assert np.array_equal(to_host(d_kc), kc) and np.array_equal(to_host(d_vc), vc)
    out1 = to_host(d_o1)
    check_attention(out1, q1_r, kc, vc, 512, 511, dt)
    bad, _ = orc.all_close(orc.widen(out1, dt), orc.attention_f32(q1_r, kc, vc, 512, 511, dt))
    assert bad == 0


def test_llama2_decode_config_fp16():
    """Benchmark configuration 2: one query token over a 512-row fp16 cache, H = Hkv = 32."""
    ops = _ops()
    dt, H, n = DT_FLOAT16, 32, 512
    q = normal_bits(2001, (1, H, 128), dt)
    k = normal_bits(2002, (n, H, 128), dt)
    v = normal_bits(2003, (n, H, 128), dt)
    d_out = dev_empty(q.shape)
    ops.hip_flash_attn_layer(d_out, to_dev(q), to_dev(k), to_dev(v), 1, n, n - 1, H, 128, dt)
    check_attention(to_host(d_out), q, k, v, n, n - 1, dt)


@pytest.mark.parametrize("dt", [DT_FLOAT16, DT_BFLOAT16])
@pytest.mark.parametrize("splits", [1, 2, 3, 7, 64, 0])
@pytest.mark.parametrize("batch,n,stride,H,Hkv", [(1, 1000, 1000, 40, 8), (3, 777, 1024, 12, 2), (2, 4096, 4096, 28, 4)])
def test_flash_decode_splits(dt, splits, batch, n, stride, H, Hkv):
    """Split-KV == unsplit for every split count incl. a ragged last split, batch
    entries independent, rows beyond n never read into the result."""
    import torch
    ops = _ops()
    q = normal_bits(31, (batch, 1, H, 128), dt)
    k = normal_bits(32, (batch, stride, Hkv, 128), dt)
    v = normal_bits(33, (batch, stride, Hkv, 128), dt)
    # poison the rows past n with NaN bit patterns: they must not reach the output
    k[:, n:] = 0x7FFF
    v[:, n:] = 0x7FFF
    g = H // Hkv
    ns = splits if splits > 0 else ops.flash_decode_default_splits(batch, n, Hkv)
    ws_bytes = ops.flash_decode_workspace_bytes(batch, g, Hkv, 128, ns)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")
    d_out = dev_empty((batch, 1, H, 128))
    ops.hip_flash_decode_gqa_layer(d_out, to_dev(q), to_dev(k), to_dev(v), ws, ws_bytes, batch, n,
                                   stride, g, Hkv, 128, splits, dt)
    check_attention(to_host(d_out), q, k, v, n, n - 1, dt, batch=True)


@pytest.mark.parametrize("S,rows_per_probe", [(1024, 24), (2400, 24), (4096, 16), (8192, 12)])
def test_qwen7b_prefill_full_size_sampled(S, rows_per_probe):
    """Benchmark configuration 4 shape (H=28, Hkv=4, bf16) at sizes the CPU oracle cannot
    finish whole: every sampled output row is checked against the oracle run as a
    one-row decode over the same keys (row r of a causal prefill == decode with
    n = r + 1)."""
    ops = _ops()
    dt, H, Hkv = DT_BFLOAT16, 28, 4
    q = normal_bits(1004 + S, (S, H, 128), dt)
    k = normal_bits(2004 + S, (S, Hkv, 128), dt)
    v = normal_bits(3004 + S, (S, Hkv, 128), dt)
    d_out = dev_empty(q.shape)
    ops.hip_flash_attn_gqa_layer(d_out, to_dev(q), to_dev(k), to_dev(v), S, S, 0, H // Hkv, Hkv, 128, dt)
    out = to_host(d_out)
    rng = np.random.default_rng(5)
    rows = sorted(set([0, 1, 31, 32, 63, 64, 255, 256, S - 1] + list(rng.integers(0, S, rows_per_probe))))
    worst = 0.0
    for r in rows:
        ref = orc.attention_f32(q[r:r + 1], k, v, r + 1, r, dt)
        err = float(np.abs(orc.widen(out[r:r + 1], dt) - ref).max())
        worst = max(worst, err)
        assert err <= TOL[dt], f"row {r}: {err}"
    assert np.isfinite(orc.widen(out, dt)).all()


@pytest.mark.parametrize("is_neox", [True, False])
def test_qwen15b_config_prefill_then_256_decode_steps(is_neox):
    """Benchmark configuration 3: Qwen2.5-1.5B, H=12, Hkv=2, bf16, theta 1e6 (table rounded to bf16,
    src/model_base.cpp:59-66), neox RoPE as the Qwen recipes run it (scripts/benchmark_qwen2.5.sh:12) and
    also interleaved, QKV bias ~ N(0, 0.02) in fp32 added before the single
    rounding to bf16 (the projection epilogue, tests/gemm_test.cpp:138-149); prefill of 256 tokens,
    then 256 decode steps with the KV cache growing in place 256 -> 512.  Every step runs the fused
    rope + append and the attention entry point; every step is checked against the oracle."""
    ops = _ops()
    dt, H, Hkv, max_seq = DT_BFLOAT16, 12, 2, 512
    rng = np.random.default_rng(1003)
    table = orc.init_freq_cis(128, max_seq, 1e6, dt)
    d_table = f32_dev(table)
    bias = {name: (rng.standard_normal(h * 128, dtype=np.float32) * np.float32(0.02)) for name, h in
            (("q", H), ("k", Hkv), ("v", Hkv))}

    def projected(m, heads, name):
        pre = orc.widen(orc.round_to(rng.standard_normal((m, heads * 128), dtype=np.float32), dt), dt)
        return orc.round_to(pre + bias[name][None, :], dt).reshape(m, heads, 128)

    kc = np.zeros((max_seq, Hkv, 128), dtype=np.uint16)
    vc = np.zeros_like(kc)
    d_kc, d_vc = to_dev(kc), to_dev(vc)
    prev, worst = 0, 0.0
    for step in range(257):
        m = 256 if step == 0 else 1
        cur = prev + m
        q, k, v = projected(m, H, "q"), projected(m, Hkv, "k"), projected(m, Hkv, "v")
        d_q, d_o = dev_empty((m, H, 128)), dev_empty((m, H, 128))
        ops.hip_rope_kv_append_layer(d_q, d_kc, d_vc, d_table, to_dev(q), to_dev(k), to_dev(v), prev, m, H,
                                     Hkv, 128, is_neox, dt)
        ops.hip_flash_attn_gqa_layer(d_o, d_q, d_kc, d_vc, m, cur, prev, H // Hkv, Hkv, 128, dt)
        q_r = orc.rope(q, table, prev, is_neox, dt)
        orc.kv_append(kc, orc.rope(k, table, prev, is_neox, dt), prev)
        orc.kv_append(vc, v, prev)
        ref = orc.attention_f32(q_r, kc, vc, cur, prev, dt)
        err = float(np.abs(orc.widen(to_host(d_o), dt) - ref).max())
        worst = max(worst, err)
        assert err <= TOL[dt], f"step {step}: {err}"
        prev = cur
    assert prev == 512
    assert np.array_equal(to_host(d_kc), kc) and np.array_equal(to_host(d_vc), vc)


@pytest.mark.parametrize("batch,n", [(1, 4096), (1, 16384), (1, 32768), (16, 4096), (16, 16384), (16, 32768)])
def test_qwen32b_decode_full_size(batch, n):
    """Benchmark configuration 5 (H=40, Hkv=8, bf16), every KV length and batch size of the benchmark, at
    full size.  The CPU oracle streams the same caches (all sequences up to 256 MiB of K+V per launch,
    sequences 0, 7 and 15 of the larger ones); plus two size-independent properties: the result does
    not depend on the split count, and (up to 256 MiB) a joint permutation of the (K, V) rows leaves
    the output unchanged up to rounding."""
    import torch
    ops = _ops()
    dt, H, Hkv = DT_BFLOAT16, 40, 8
    g = H // Hkv
    q = normal_bits(1005, (batch, 1, H, 128), dt)
    # the caches are generated one sequence at a time (a 2 GiB launch would need 8 GiB of fp32 normals)
    k = np.empty((batch, n, Hkv, 128), dtype=np.uint16)
    v = np.empty_like(k)
    for b in range(batch):
        k[b] = normal_bits(1006 + 2 * b, (n, Hkv, 128), dt)
        v[b] = normal_bits(1007 + 2 * b, (n, Hkv, 128), dt)
    dk, dv = to_dev(k), to_dev(v)
    dq = to_dev(q)

    def run(d_k, d_v, splits):
        ns = splits if splits > 0 else ops.flash_decode_default_splits(batch, n, Hkv)
        wsb = ops.flash_decode_workspace_bytes(batch, g, Hkv, 128, ns)
        ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda")
        d_out = dev_empty((batch, 1, H, 128))
        ops.hip_flash_decode_gqa_layer(d_out, dq, d_k, d_v, ws, wsb, batch, n, n, g, Hkv, 128, splits, dt)
        return to_host(d_out)

    out = run(dk, dv, 0)
    small = 2 * k.nbytes <= 256 << 20
    if small:
        check_attention(out, q, k, v, n, n - 1, dt, batch=True)
    else:
        for b in sorted({0, 7 % batch, batch - 1}):
            check_attention(out[b], q[b], k[b], v[b], n, n - 1, dt)
    out_s = run(dk, dv, 7)
    assert np.abs(orc.widen(out, dt) - orc.widen(out_s, dt)).max() <= 2 * 2.0 ** -8
    if small:
        perm = np.random.default_rng(9).permutation(n)
        out_p = run(to_dev(np.ascontiguousarray(k[:, perm])), to_dev(np.ascontiguousarray(v[:, perm])), 0)
        assert np.abs(orc.widen(out, dt) - orc.widen(out_p, dt)).max() <= 2 * 2.0 ** -8


CHUNK_CASES = [
    # (m, n, offset, H, Hkv): few query rows over a long cache -> the key range is split over workgroups
    (64, 8256, 8192, 28, 4),      # 128-row kernel, every row sees every range
    (200, 5000, 4800, 28, 4),     # 256-row kernel (m >= 192), ragged last range
    (256, 33024, 32768, 28, 4),   # the chunked-prefill benchmark shape
    (100, 9000, 9500, 8, 2),      # n < m + offset: the cache length cuts every row
    (17, 4099, 4082, 5, 1),       # one 128-row tile, one active wave, odd sizes
    (40, 20000, 19960, 40, 8),    # Qwen2.5-32B head counts: 200 packed rows per kv head, 256-row kernel
    (8, 6000, 5992, 28, 4),       # 56 packed rows: one 128-row tile per kv head
    (20, 3000, 2980, 12, 2),      # 120 packed rows, g = 6
    (127, 16384, 16257, 14, 2),   # 889 packed rows: four 256-row tiles per kv head, ragged last tile
    (33, 2500, 2467, 3, 3),       # g = 1: nothing to pack
]


@pytest.mark.parametrize("dt", [DT_FLOAT16, DT_BFLOAT16])
@pytest.mark.parametrize("m,n,offset,H,Hkv", CHUNK_CASES)
def test_chunked_prefill_key_split_vs_oracle(dt, m, n, offset, H, Hkv):
    """A chunk of m new tokens over a cache of n >> m keys (chunked prefill): the prefill kernel splits the
    key range over workgroups and folds the fp32 partials (log-sum-exp).  Rows past n are poisoned."""
    ops = _ops()
    seed = 500 * m + n + H
    q = normal_bits(seed, (m, H, 128), dt)
    k = normal_bits(seed + 1, (n + 5, Hkv, 128), dt)
    v = normal_bits(seed + 2, (n + 5, Hkv, 128), dt)
    k[n:] = 0x7FFF
    v[n:] = 0x7FFF
    d_out = dev_empty(q.shape)
    ops.hip_flash_attn_gqa_layer(d_out, to_dev(q), to_dev(k), to_dev(v), m, n, offset, H // Hkv, Hkv, 128, dt)
    check_attention(to_host(d_out), q, k, v, n, offset, dt)


def test_long_context_131072():
    """A 131072-token cache (the longest context Qwen2.5 advertises) at the 32B head counts: one decode
    step and a 40-token chunk appended at the end (the prefill kernel walking 2048 key tiles), against
    the oracle.  Guards the 32/64-bit address arithmetic of both kernels."""
    ops = _ops()
    dt, H, Hkv, n = DT_BFLOAT16, 40, 8, 131072
    k = normal_bits(1301, (n, Hkv, 128), dt)
    v = normal_bits(1302, (n, Hkv, 128), dt)
    dk, dv = to_dev(k), to_dev(v)
    for m in (1, 40):
        # (a seed of its own: with the seed of k the first query row would equal key 0 and give a row
        # peaked on one key, which the layer-style bf16 chain itself resolves only to ~2e-2)
        q = normal_bits(1310 + m, (m, H, 128), dt)
        d_out = dev_empty(q.shape)
        ops.hip_flash_attn_gqa_layer(d_out, to_dev(q), dk, dv, m, n, n - m, H // Hkv, Hkv, 128, dt)
        check_attention(to_host(d_out), q, k, v, n, n - m, dt)


@pytest.mark.parametrize("dt", [DT_BFLOAT16, DT_FLOAT16])
def test_short_chunk_over_131072_keys_two_kv_heads(dt):
    """The Qwen2.5-1.5B head counts (12 query heads on 2 kv heads): 9 new tokens over a 131072-key cache run
    as 54 packed rows per kv head over 128 key ranges, each K/V tile read by one workgroup (non-temporal
    loads), folded by the combine kernel for few rows and many ranges."""
    ops = _ops()
    H, Hkv, n, m = 12, 2, 131072, 9
    q = normal_bits(1410, (m, H, 128), dt)
    k = normal_bits(1411, (n + 2, Hkv, 128), dt)
    v = normal_bits(1412, (n + 2, Hkv, 128), dt)
    k[n:] = 0x7FFF
    v[n:] = 0x7FFF
    assert ops.lib.llmhip_flash_attn_scratch_bytes(m, n, n - m, H // Hkv, Hkv) == 128 * m * H * 130 * 4
    d_out = dev_empty(q.shape)
    ops.hip_flash_attn_gqa_layer(d_out, to_dev(q), to_dev(k), to_dev(v), m, n, n - m, H // Hkv, Hkv, 128, dt)
    check_attention(to_host(d_out), q, k, v, n, n - m, dt)


def test_flash_decode_random_shapes():
    """Seeded sweep of the batched decode entry point: batch, KV length, allocated rows per sequence, group
    size and kv heads drawn at random (group sizes up to the 16 columns of the kernel), default splits."""
    import torch
    ops = _ops()
    rng = np.random.default_rng(20250101)
    for i in range(24):
        dt = DT_BFLOAT16 if i % 2 else DT_FLOAT16
        batch = int(rng.integers(1, 6))
        n = int(rng.choice([1, 2, 31, 32, 33, 127, 128, 129, int(rng.integers(130, 3000))]))
        stride = n + int(rng.choice([0, 1, 17]))
        g = int(rng.choice([1, 2, 3, 5, 7, 8, 16]))
        Hkv = int(rng.choice([1, 2, 3, 8]))
        H = g * Hkv
        q = normal_bits(9000 + i, (batch, 1, H, 128), dt)
        k = normal_bits(9100 + i, (batch, stride, Hkv, 128), dt)
        v = normal_bits(9200 + i, (batch, stride, Hkv, 128), dt)
        k[:, n:] = 0x7FFF
        v[:, n:] = 0x7FFF
        wsb = ops.flash_decode_workspace_bytes(batch, g, Hkv, 128, 0)
        ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda")
        d_out = dev_empty((batch, 1, H, 128))
        ops.hip_flash_decode_gqa_layer(d_out, to_dev(q), to_dev(k), to_dev(v), ws, wsb, batch, n, stride, g, Hkv,
                                       128, 0, dt)
        check_attention(to_host(d_out), q, k, v, n, n - 1, dt, batch=True)


def test_attention_random_shapes():
    """Seeded sweep of the reference-signature attention entry point over the four regimes of its dispatch:
    square causal prefill (all kernel shapes for short sequences), a chunk of few rows over a long cache
    (key-range split, packed rows), decode-sized calls (m * group_size <= 16), and ragged cases where the
    cache length cuts the rows.  Rows past n are poisoned."""
    import random
    ops = _ops()
    rnd = random.Random(20251125)
    for it in range(48):
        Hkv = rnd.choice([1, 2, 3, 4, 8])
        g = rnd.choice([1, 1, 2, 5, 6, 7, 16])
        H = Hkv * g
        kind = ("square", "chunk", "decode", "ragged")[it % 4]
        if kind == "square":
            m = rnd.randint(1, 700)
            n, off = m, 0
        elif kind == "chunk":
            m = rnd.randint(1, 130)
            n = rnd.randint(2048, 9000)
            off = n - m
        elif kind == "decode":
            m = rnd.randint(1, max(1, 16 // g))
            n = rnd.randint(1, 6000)
            off = max(0, n - m)
        else:
            m = rnd.randint(1, 300)
            off = rnd.randint(0, 500)
            n = rnd.randint(1, m + off + 50)
        dt = DT_BFLOAT16 if rnd.random() < 0.5 else DT_FLOAT16
        q = normal_bits(17000 + it, (m, H, 128), dt)
        k = normal_bits(18000 + it, (n + 3, Hkv, 128), dt)
        v = normal_bits(19000 + it, (n + 3, Hkv, 128), dt)
        k[n:] = 0x7FFF
        v[n:] = 0x7FFF
        d_out = dev_empty(q.shape)
        print(f"case {it}: {kind} m={m} n={n} offset={off} H={H} Hkv={Hkv} dt={dt}", flush=True)
        ops.hip_flash_attn_gqa_layer(d_out, to_dev(q), to_dev(k), to_dev(v), m, n, off, g, Hkv, 128, dt)
        check_attention(to_host(d_out), q, k, v, n, off, dt)


@pytest.mark.parametrize("dt", [DT_FLOAT16, DT_BFLOAT16])
@pytest.mark.parametrize("is_neox", [False, True])
@pytest.mark.parametrize("H,Hkv", [(12, 2), (32, 32), (40, 8), (28, 4)])
def test_decode_step_fused_equals_unfused_chain(dt, is_neox, H, Hkv):
    """llmhip_decode_step_gqa (rope + append inside the decode kernel) against the unfused sequence
    rope_kv_append -> flash_attn_gqa(m=1): output, K-cache row and V-cache row bit-identical, at cache
    lengths around every boundary of the kernel (one key, a 32-key wave step, a 128-key workgroup step, a
    split boundary, many splits); untouched rows keep their bytes; and the output against the oracle."""
    ops = _ops()
    max_seq = 5000
    theta = 1e6 if dt == DT_BFLOAT16 else 10000.0
    table = orc.init_freq_cis(128, max_seq, theta, dt)
    d_table = f32_dev(table)
    kc0 = normal_bits(61, (max_seq, Hkv, 128), dt)
    vc0 = normal_bits(62, (max_seq, Hkv, 128), dt)
    for pos in (0, 1, 31, 32, 127, 128, 129, 1000, 4095, 4999):
        q = normal_bits(7000 + pos, (1, H, 128), dt)
        k = normal_bits(7100 + pos, (1, Hkv, 128), dt)
        v = normal_bits(7200 + pos, (1, Hkv, 128), dt)
        # unfused
        kc_a, vc_a = to_dev(kc0), to_dev(vc0)
        qe, o_a = dev_empty(q.shape), dev_empty(q.shape)
        ops.hip_rope_kv_append_layer(qe, kc_a, vc_a, d_table, to_dev(q), to_dev(k), to_dev(v), pos, 1, H, Hkv, 128,
                                     is_neox, dt)
        ops.hip_flash_attn_gqa_layer(o_a, qe, kc_a, vc_a, 1, pos + 1, pos, H // Hkv, Hkv, 128, dt)
        # fused
        kc_b, vc_b = to_dev(kc0), to_dev(vc0)
        o_b = dev_empty(q.shape)
        ops.hip_decode_step_gqa_layer(o_b, kc_b, vc_b, d_table, to_dev(q), to_dev(k), to_dev(v), pos, H // Hkv, Hkv,
                                      128, is_neox, dt)
        assert np.array_equal(to_host(kc_b), to_host(kc_a)), f"K cache differs at pos {pos}"
        assert np.array_equal(to_host(vc_b), to_host(vc_a)), f"V cache differs at pos {pos}"
        assert np.array_equal(to_host(o_b), to_host(o_a)), f"output differs at pos {pos}"
        if pos in (0, 129, 4999):
            kc_h, vc_h = to_host(kc_b), to_host(vc_b)
            check_attention(to_host(o_b), orc.rope(q, table, pos, is_neox, dt), kc_h, vc_h, pos + 1, pos, dt)
