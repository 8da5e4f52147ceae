#!/usr/bin/env python3
"""Writes tests/golden/attention_golden.npz: small input/output vectors of the hot path
produced by THIS repository's CPU oracle (oracle/attn_oracle.c), not by the reference
(whose sources cannot be built here and whose tests keep no vectors on disk).  They
freeze the oracle's behaviour: a later change of the oracle or of the kernels that
moves any of these numbers shows up as a test failure.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as orc  # noqa: E402

CASES = [(4, 4, 0, 2, 2), (3, 7, 4, 4, 2), (1, 33, 32, 6, 1)]  # (m, n, offset, H, Hkv)


def bits(seed, shape, dt):
    rng = np.random.default_rng(seed)
    return orc.round_to(rng.standard_normal(shape, dtype=np.float32), dt)


def main():
    out = {}
    for theta in (1e4, 1e6):
        for dt in (orc.DT_FLOAT16, orc.DT_BFLOAT16):
            tab = orc.init_freq_cis(128, 32768, theta, dt)
            out[f"freq_theta{int(theta)}_dt{dt}"] = tab[[0, 1, 511, 32767]]
    for ci, (m, n, offset, H, Hkv) in enumerate(CASES):
        for dt in (orc.DT_FLOAT16, orc.DT_BFLOAT16):
            theta = 1e4 if dt == orc.DT_FLOAT16 else 1e6
            tab = orc.init_freq_cis(128, 64, theta, dt)
            q, k, v = bits(10 * ci + 1, (m, H, 128), dt), bits(10 * ci + 2, (m, Hkv, 128), dt), bits(10 * ci + 3, (m, Hkv, 128), dt)
            k_old, v_old = bits(10 * ci + 4, (n - m, Hkv, 128), dt), bits(10 * ci + 5, (n - m, Hkv, 128), dt)
            key = f"c{ci}_dt{dt}"
            out[key + "_q"], out[key + "_k"], out[key + "_v"] = q, k, v
            out[key + "_k_old"], out[key + "_v_old"] = k_old, v_old
            for neox in (0, 1):
                q_r = orc.rope(q, tab, offset, neox, dt)
                kc = np.zeros((n, Hkv, 128), dtype=np.uint16)
                vc = np.zeros((n, Hkv, 128), dtype=np.uint16)
                kc[:n - m], vc[:n - m] = k_old, v_old
                orc.kv_append(kc, orc.rope(k, tab, offset, neox, dt), n - m)
                orc.kv_append(vc, v, n - m)
                out[f"{key}_neox{neox}_q_rope"] = q_r
                out[f"{key}_neox{neox}_k_cache"] = kc
                out[f"{key}_neox{neox}_v_cache"] = vc
                out[f"{key}_neox{neox}_out_f32"] = orc.attention_f32(q_r, kc, vc, n, offset, dt)
                out[f"{key}_neox{neox}_out_layer"] = orc.attention_layer(q_r, kc, vc, n, offset, dt)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "attention_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
