"""Committed golden vectors (tests/golden/attention_golden.npz, written by
tests/golden/make_golden.py from this repository's oracle): the oracle must still
reproduce them bit for bit (CPU), and the HIP path must match them on the GPU --
RoPE and both caches bit for bit, the attention output within the tolerance."""
import os

import numpy as np
import pytest

from helpers import TOL, dev_empty, f32_dev, to_dev, to_host
from oracle import oracle as orc

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "attention_golden.npz"))
CASES = [(4, 4, 0, 2, 2), (3, 7, 4, 4, 2), (1, 33, 32, 6, 1)]


def test_freq_rows_reproduce():
    for theta in (1e4, 1e6):
        for dt in (orc.DT_FLOAT16, orc.DT_BFLOAT16):
            tab = orc.init_freq_cis(128, 32768, theta, dt)
            assert np.array_equal(tab[[0, 1, 511, 32767]], G[f"freq_theta{int(theta)}_dt{dt}"])


@pytest.mark.parametrize("ci", range(3))
@pytest.mark.parametrize("dt", [orc.DT_FLOAT16, orc.DT_BFLOAT16])
@pytest.mark.parametrize("neox", [0, 1])
def test_oracle_reproduces_golden(ci, dt, neox):
    m, n, offset, H, Hkv = CASES[ci]
    key = f"c{ci}_dt{dt}"
    tab = orc.init_freq_cis(128, 64, 1e4 if dt == orc.DT_FLOAT16 else 1e6, dt)
    q_r = orc.rope(G[key + "_q"], tab, offset, neox, dt)
    assert np.array_equal(q_r, G[f"{key}_neox{neox}_q_rope"])
    kc, vc = G[f"{key}_neox{neox}_k_cache"], G[f"{key}_neox{neox}_v_cache"]
    assert np.array_equal(orc.rope(G[key + "_k"], tab, offset, neox, dt), kc[n - m:])
    assert np.array_equal(orc.attention_f32(q_r, kc, vc, n, offset, dt), G[f"{key}_neox{neox}_out_f32"])
    assert np.array_equal(orc.attention_layer(q_r, kc, vc, n, offset, dt), G[f"{key}_neox{neox}_out_layer"])


@pytest.mark.gpu
@pytest.mark.parametrize("ci", range(3))
@pytest.mark.parametrize("dt", [orc.DT_FLOAT16, orc.DT_BFLOAT16])
@pytest.mark.parametrize("neox", [0, 1])
def test_hip_path_matches_golden(ci, dt, neox):
    import llm_simple_amd.ops as ops
    m, n, offset, H, Hkv = CASES[ci]
    key = f"c{ci}_dt{dt}"
    tab = orc.init_freq_cis(128, 64, 1e4 if dt == orc.DT_FLOAT16 else 1e6, dt)
    kc = np.zeros((n, Hkv, 128), dtype=np.uint16)
    vc = np.zeros((n, Hkv, 128), dtype=np.uint16)
    kc[:n - m], vc[:n - m] = G[key + "_k_old"], G[key + "_v_old"]
    d_q, d_kc, d_vc = dev_empty((m, H, 128)), to_dev(kc), to_dev(vc)
    ops.hip_rope_kv_append_layer(d_q, d_kc, d_vc, f32_dev(tab), to_dev(G[key + "_q"]), to_dev(G[key + "_k"]),
                                 to_dev(G[key + "_v"]), offset, m, H, Hkv, 128, bool(neox), dt)
    d_o = dev_empty((m, H, 128))
    ops.hip_flash_attn_gqa_layer(d_o, d_q, d_kc, d_vc, m, n, offset, H // Hkv, Hkv, 128, dt)
    assert np.array_equal(to_host(d_q), G[f"{key}_neox{neox}_q_rope"])
    assert np.array_equal(to_host(d_kc), G[f"{key}_neox{neox}_k_cache"])
    assert np.array_equal(to_host(d_vc), G[f"{key}_neox{neox}_v_cache"])
    err = np.abs(orc.widen(to_host(d_o), dt) - G[f"{key}_neox{neox}_out_f32"]).max()
    assert err <= TOL[dt], err
