"""Pins the three rounding points of the layer-style oracle (orc_attention_layer), the restatement
of the reference CPU attention: scores rounded to the storage type T after the scale
(src/llama2_layer_cpu.cpp:218-219), probabilities rounded to T after the division by the row sum
(src/llama2_layer_cpu.cpp:675), output rounded to T after the fp32 contraction (:275-279).

Every case is one head, one query row, two to eleven keys, with inputs made of small integers and
powers of two so that each dot product is exact in fp32 in any summation order; the expected
outputs are bit patterns written out below with their derivation.  The value rows are unit vectors
(plus one or two combination columns), so the output exposes the probabilities themselves.

`_model` is an independent float64 evaluation with switchable rounding points.  It is used for two
things only: to confirm the hand-derived literals, and to show that every wrong chain (a rounding
dropped, moved before the division, or done in the other 16-bit type) misses at least one literal,
i.e. that these cases can fail."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc

F16, BF16 = orc.DT_FLOAT16, orc.DT_BFLOAT16
SCALE32 = np.float32(1.0) / np.sqrt(np.float32(128.0))  # 1/sqrtf(128), src/llama2_layer_cpu.cpp:177


def _bits(x, dt):
    """float32 array -> bits of the storage type, through the library casts (not the oracle's)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    if dt == F16:
        return x.astype(np.float16).view(np.uint16)
    return torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def _rows(rows, dt):
    a = np.zeros((len(rows), 1, 128), dtype=np.float32)
    for i, r in enumerate(rows):
        a[i, 0, :len(r)] = r
    b = _bits(a, dt)
    assert np.array_equal(orc.widen(b, dt), a), "inputs must be exactly representable"
    return b


def _layer(q_row, k_rows, v_rows, dt, width):
    n = len(k_rows)
    out = orc.attention_layer(_rows([q_row], dt), _rows(k_rows, dt), _rows(v_rows, dt), n, n - 1, dt)
    return [int(x) for x in out.reshape(-1)[:width]]


def _f32(q_row, k_rows, v_rows, dt, width):
    n = len(k_rows)
    out = orc.attention_f32(_rows([q_row], dt), _rows(k_rows, dt), _rows(v_rows, dt), n, n - 1, dt)
    return out.reshape(-1)[:width]


# ---------------------------------------------------------------- the cases
# q = (1, 1, 1, 0, ...): the dot product with key (a, b, c, 0, ...) is a + b + c exactly.
Q = [1.0, 1.0, 1.0]
# value rows: unit vector of the key, and a last column of +1 / -1 (two-key cases)
V2 = [[1.0, 0.0, 1.0], [0.0, 1.0, -1.0]]

# Case A: dots 150 and 150.25.  Raw scores fl32(dot * scale) = 13.258252, 13.280349.
#   bf16 (steps of 2^-4 in [8,16)): both fall in the cell [13.21875, 13.28125] of 13.25 -> equal
#     scores -> P = (1/2, 1/2) exactly -> out = (0.5, 0.5, 0) = 3f00 3f00 0000.
#   fp16 (steps of 2^-7): 13.2578125 and 13.28125, apart by 3 * 2^-7 = 0.0234375 ->
#     P1 = 1/(1+e^-0.0234375) = 0.50585911 -> 1036 * 2^-11 = 380c; P0 = 0.49414089 -> 2024 * 2^-12 =
#     37e8; out[2] = P0 - P1 = (2024 - 2072)/4096 = -48/4096 = -0.01171875 = a200.
CASE_A = dict(k=[[150.0, 0.0, 0.0], [150.0, 0.25, 0.0]], v=V2,
              want={BF16: [0x3F00, 0x3F00, 0x0000], F16: [0x37E8, 0x380C, 0xA200]})
# Case B: dots 363 = 256 + 107 and 363.25.  Raw scores 32.084969, 32.107067: fp16 has steps of 2^-5
#   in [32,64): both in the cell of 32.09375; bf16 (steps of 2^-2): both 32.0 -> P = (1/2, 1/2).
CASE_B = dict(k=[[256.0, 107.0, 0.0], [256.0, 107.0, 0.25]], v=V2,
              want={BF16: [0x3F00, 0x3F00, 0x0000], F16: [0x3800, 0x3800, 0x0000]})
# Case C: dots 11.3125 and 0: raw scores 0.9998932 and 0; rounded (either type) 1.0 and 0.
#   e = (1, exp(-1)), sum 1.3678794; P0 = 0.73105858, P1 = 0.26894142.
#   fp16: P0 -> 1497 * 2^-11 = 39d9, P1 -> 1102 * 2^-12 = 344e (1101.58 rounds up);
#         out[2] = P0 - P1 = (2994 - 1102)/4096 = 1892 * 2^-12 = 3764.
#         Without the rounding of P: 0.46211716 -> 1893 * 2^-12 = 3765.
#   bf16: P0 -> 187 * 2^-8 = 3f3b, P1 -> 138 * 2^-9 = 3e8a (137.70 rounds up);
#         out[2] = (374 - 138)/512 = 236 * 2^-9 = 3eec.  Without the rounding of P: 236.6 -> 3eed.
#         Rounding exp(-1) -> 188 * 2^-9 BEFORE the division gives P1 = 0.26843566 -> 137 * 2^-9 = 3e89.
CASE_C = dict(k=[[11.0, 0.25, 0.0625], [0.0, 0.0, 0.0]], v=V2,
              want={BF16: [0x3F3B, 0x3E8A, 0x3EEC], F16: [0x39D9, 0x344E, 0x3764]})


def _equal_keys(n):
    # n identical keys (dot 5): P = 1/n each; value row c = (1, unit vector c)
    return dict(k=[[5.0, 0.0, 0.0]] * n, v=[[1.0] + [1.0 if j == c else 0.0 for j in range(n)] for c in range(n)])


# Case D11 (fp16): 11 equal keys.  1/11 -> 1489 * 2^-14 = 2dd1 (1489.45 rounds down);
#   out[0] = 11 * 1489 * 2^-14 = 16379 * 2^-14 = 1 - 5 * 2^-14, between 3bff (1 - 8 * 2^-14) and 3c00:
#   nearer 3bff.  With unrounded probabilities the sum is 1.0 = 3c00.
CASE_D11 = dict(_equal_keys(11), want={F16: [0x3BFF] + [0x2DD1] * 11})
# Case D3 (fp16): 3 equal keys.  1/3 -> 2730 * 2^-13 = 3555; out[0] = 8190 * 2^-13 = 1 - 2^-12,
#   exactly halfway between 3bff and 3c00: nearest-even gives 3c00 (truncation would give 3bff).
CASE_D3 = dict(_equal_keys(3), want={F16: [0x3C00] + [0x3555] * 3, BF16: [0x3F80] + [0x3EAB] * 3})

CASES = {"A": CASE_A, "B": CASE_B, "C": CASE_C, "D11": CASE_D11, "D3": CASE_D3}
ALL = [(name, dt) for name, c in CASES.items() for dt in c["want"]]


@pytest.mark.parametrize("name,dt", ALL)
def test_layer_oracle_reproduces_hand_derived_bits(name, dt):
    c = CASES[name]
    want = c["want"][dt]
    got = _layer(Q, c["k"], c["v"], dt, len(want))
    assert got == want, f"case {name}: got {[hex(x) for x in got]}, want {[hex(x) for x in want]}"


def test_f32_oracle_does_not_round_the_scores():
    """The fp32 golden (tests/flash_attn_test.cpp:106-192) keeps the two scores of cases A and B
    apart: it must NOT return the collapsed (1/2, 1/2)."""
    for c, dt in ((CASE_A, BF16), (CASE_B, F16), (CASE_B, BF16)):
        o = _f32(Q, c["k"], c["v"], dt, 3)
        assert o[0] < 0.4999 and o[1] > 0.5001 and o[2] < -1e-3
    # A: difference of raw scores 0.25 * scale = 0.0220971 -> P1 - P0 = tanh(0.0220971 / 2)
    o = _f32(Q, CASE_A["k"], CASE_A["v"], F16, 3)
    assert abs(float(o[1] - o[0]) - np.tanh(0.25 * float(SCALE32) / 2)) < 2e-6


# ---------------------------------------------------------------- the cases can fail

def _model(c, dt, round_scores=True, probs="after", score_dt=None):
    """float64 arithmetic with library casts at the rounding points."""
    def rt(x, t):
        b = _bits(np.asarray(x, dtype=np.float32), t)
        w = b.view(np.float16).astype(np.float32) if t == F16 else (b.astype(np.uint32) << 16).view(np.float32)
        return w.astype(np.float64)
    dots = np.array([sum(r) for r in c["k"]], dtype=np.float64)  # q = ones on the first three dims
    s = (dots * np.float64(SCALE32)).astype(np.float32)
    if round_scores:
        s = rt(s, score_dt or dt).astype(np.float32)
    e = np.exp((s - s.max()).astype(np.float64))
    if probs == "after":
        p = rt(e / e.sum(), dt)
    elif probs == "before":
        p = rt(e, dt) / e.sum()
    else:
        p = e / e.sum()
    o = (p[:, None] * np.asarray(c["v"], dtype=np.float64)).sum(0)
    return [int(x) for x in _bits(o, dt)]


def test_model_confirms_the_literals():
    for name, dt in ALL:
        c = CASES[name]
        assert _model(c, dt) == c["want"][dt], (name, dt)


@pytest.mark.parametrize("mutant", [dict(round_scores=False), dict(probs="none"), dict(probs="before"),
                                    dict(score_dt="other")])
def test_every_wrong_chain_misses_a_literal(mutant):
    """For each dtype, a chain without the score rounding, without the probability rounding, with the
    probabilities rounded before the division, or with the scores rounded to the other 16-bit type
    disagrees with at least one expected bit pattern."""
    for dt in (F16, BF16):
        kw = dict(mutant)
        if kw.get("score_dt") == "other":
            kw["score_dt"] = BF16 if dt == F16 else F16
        misses = [name for name, d in ALL if d == dt and _model(CASES[name], dt, **kw) != CASES[name]["want"][dt]]
        assert misses, f"dt {dt}: mutant {mutant} passes every case"
