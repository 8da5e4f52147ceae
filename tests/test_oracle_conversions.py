"""Pins the oracle's storage-type conversions and rotary table without running
the reference: exhaustive round trips, library casts, closed forms."""
import numpy as np
import torch

from oracle import oracle as orc

F16, BF16 = orc.DT_FLOAT16, orc.DT_BFLOAT16


def test_f16_round_trip_exhaustive():
    bits = np.arange(1 << 16, dtype=np.uint16)
    wide = orc.widen(bits, F16)
    lib = bits.view(np.float16).astype(np.float32)
    finite = np.isfinite(lib)
    assert np.array_equal(wide[finite], lib[finite])
    assert np.array_equal(np.isnan(wide), np.isnan(lib))
    back = orc.round_to(wide, F16)
    assert np.array_equal(back[~np.isnan(lib)], bits[~np.isnan(lib)])


def test_bf16_round_trip_exhaustive():
    bits = np.arange(1 << 16, dtype=np.uint16)
    wide = orc.widen(bits, BF16)
    assert np.array_equal(wide.view(np.uint32), bits.astype(np.uint32) << 16)
    keep = np.isfinite(wide)
    assert np.array_equal(orc.round_to(wide, BF16)[keep], bits[keep])


def test_f16_rounding_matches_numpy():
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32),
        (rng.standard_normal(50000) * 1e-6).astype(np.float32),   # subnormal results
        (rng.standard_normal(50000) * 3e4).astype(np.float32),    # near overflow
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25,
                  1.5 * 2.0 ** -25, 2.0 ** -14, np.inf, -np.inf], dtype=np.float32)])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.round_to(x, F16), want)


def test_f16_ties_to_even():
    # 1 + 2^-11 is exactly half way between 1 and 1 + 2^-10: even mantissa wins
    assert orc.f32_to_f16_scalar(1.0 + 2.0 ** -11) == 0x3C00
    assert orc.f32_to_f16_scalar(1.0 + 3 * 2.0 ** -11) == 0x3C02
    assert orc.f32_to_f16_scalar(1.0 + 2.0 ** -11 + 2.0 ** -20) == 0x3C01


def test_bf16_rounding_matches_torch():
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(300000).astype(np.float32),
                        (rng.standard_normal(1000) * 1e30).astype(np.float32),
                        np.array([0.0, -0.0, 1.0, np.inf, -np.inf], dtype=np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(orc.round_to(x, BF16), want)


def test_bf16_ties_to_even_bit_patterns():
    # low half == 0x8000: round to the even upper half
    assert orc.f32_to_bf16_scalar(0x3F808000) == 0x3F80
    assert orc.f32_to_bf16_scalar(0x3F818000) == 0x3F82
    assert orc.f32_to_bf16_scalar(0x3F808001) == 0x3F81
    assert orc.f32_to_bf16_scalar(0x3F807FFF) == 0x3F80
    # mantissa carry into the exponent
    assert orc.f32_to_bf16_scalar(0x3FFFFFFF) == 0x4000
    assert orc.f32_to_bf16_scalar(0xBFFFFFFF) == 0xC000


def test_freq_cis_closed_form():
    for theta in (1e4, 1e6):
        tab = orc.init_freq_cis(128, 4096, theta, F16)
        assert tab.shape == (4096, 64, 2)
        assert np.all(tab[0, :, 0] == 1.0) and np.all(tab[0, :, 1] == 0.0)
        i = np.arange(64, dtype=np.float64)
        inv = theta ** (-2.0 * i / 128.0)
        t = np.arange(4096, dtype=np.float64)[:, None]
        # the table forms the angle in fp32: allow one rounding of inv (2^-24
        # relative) and one of the product, both scaled by the angle
        ang = t * inv[None, :]
        bound = 2.0 ** -22 * np.maximum(ang, 1.0) + 1e-6
        assert np.all(np.abs(tab[..., 0] - np.cos(ang)) <= bound)
        assert np.all(np.abs(tab[..., 1] - np.sin(ang)) <= bound)
        # unit modulus
        assert np.abs(tab[..., 0].astype(np.float64) ** 2 + tab[..., 1].astype(np.float64) ** 2 - 1).max() < 1e-6


def test_freq_cis_bf16_rounding_idempotent_and_close():
    full = orc.init_freq_cis(128, 512, 1e6, F16)
    b = orc.init_freq_cis(128, 512, 1e6, BF16)
    assert np.array_equal(orc.widen(orc.round_to(b, BF16), BF16), b)     # already bf16 values
    assert np.array_equal(orc.widen(orc.round_to(full, BF16), BF16), b)  # == rounding the fp32 table
    assert np.abs(b - full).max() <= 2.0 ** -8


def test_freq_cis_test_twin_agrees_within_powf_rounding():
    a = orc.init_freq_cis(128, 2048, 1e4, F16, use_powf=False)
    b = orc.init_freq_cis(128, 2048, 1e4, BF16, use_powf=True)  # the twin never rounds to bf16
    assert np.abs(a - b).max() < 2e-3  # angle up to 2047 rad times 2^-23 relative


def test_product_table_matches_oracle_table():
    from llm_simple_amd.ops import init_freq_cis
    for theta, dt in ((1e4, F16), (1e6, BF16), (1e6, F16)):
        a = orc.init_freq_cis(128, 1024, theta, dt)
        b = init_freq_cis(128, 1024, theta, dt)
        # numpy's float32 cos/sin vs libm's cosf/sinf: at most an ulp apart,
        # one bf16 step after rounding
        tol = 2.0 ** -7 if dt == BF16 else 2.5e-7
        assert np.abs(a - b).max() <= tol
