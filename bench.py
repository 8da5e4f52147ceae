#!/usr/bin/env python3
"""Benchmark of the MI355X attention path: one JSON line on stdout.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one pass of the hot path over one batch of synthetic input that is
already resident in HBM: the causal flash-attention prefill launch at
the headline benchmark shape, Qwen2.5-7B (bf16, H=28, Hkv=4, head_dim 128, S=4096).
`value` is its algorithmic throughput, 4*H*hd*S(S+1)/2 FLOP per launch over the
measured time per launch.  The same run also measures the two other kernels of
the path at their benchmark shapes -- split-KV decode at the Qwen2.5-32B shape
(H=40, Hkv=8, KV length 32768, batch 1 and 16; algorithmic bytes = K and V read
once) and the fused RoPE + KV append -- and times the CPU oracle (a port of the
reference's CPU layer attention, src/llama2_layer_cpu.cpp:175-296) on the host
cores as a reported baseline.

Launch durations are measured with HIP events recorded on the stream the
kernels run on (the default stream), around back-to-back launches.  Whatever
--steps/--warmup say, every leg first launches for at least 100 ms so that the
clocks settle (the first ~50 ms of a burst run about 8 % slower than the
sustained rate; reported as settle_ms), then takes the median of 5 batches of
max(steps, 100) launches.  After the timed region the outputs of the timed
launches are compared with the CPU oracle on sampled rows (max_abs_err).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "attn prefill TFLOP/s + decode KV GB/s (Qwen2.5-7B shape), % roofline, 1 MI355X"
PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, published
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E, published
DT_BF16 = 5
DT_F16 = 4

# HBM bytes per launch read off rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch, FETCH_SIZE
# scaled by 2.000 and WRITE_SIZE by 1.000, the factors a plain 1 GiB copy gives); the commands and raw
# figures are in profiles/.  Only the shapes that were profiled have an entry.
TRAFFIC_SOURCE = "rocprofv3 --pmc FETCH_SIZE/WRITE_SIZE summaries under profiles/ (not measured in this run)"
MEASURED_TRAFFIC_BYTES = {
    ("prefill", 4096): (47165 + 28672) * 1024,             # algorithmic 65536 KiB
    ("decode", 16, 32768): (2097637 + 656) * 1024,         # algorithmic 2097152 KiB
    ("decode", 1, 32768): (131317 + 656) * 1024,           # algorithmic 131072 KiB
    ("rope", 4096): (40753 + 36887) * 1024,                # algorithmic 75776 KiB
    ("chunked", 256, 33024): (136014 + 33556 + 33282 + 1792) * 1024,   # prefill kernel + combine
    ("chunked", 40, 131072): (537483 + 26242 + 28843 + 400) * 1024,
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class HipTimer:
    """Event pair on the default stream through the library's own event calls."""

    def __init__(self, lib):
        import ctypes
        self.lib = lib
        self.a, self.b = ctypes.c_void_p(), ctypes.c_void_p()
        assert lib.llmhip_event_create(ctypes.byref(self.a)) == 0
        assert lib.llmhip_event_create(ctypes.byref(self.b)) == 0

    def time_ms(self, fn, reps):
        import ctypes
        assert self.lib.llmhip_event_record(self.a, None) == 0
        for i in range(reps):
            fn(i)
        assert self.lib.llmhip_event_record(self.b, None) == 0
        assert self.lib.llmhip_event_sync(self.b) == 0
        ms = ctypes.c_float(0)
        assert self.lib.llmhip_event_elapsed_ms(ctypes.byref(ms), self.a, self.b) == 0
        return ms.value / reps


def median(xs):
    xs = sorted(xs)
    return xs[len(xs) // 2]


SETTLE_MS = 100.0   # launches before any timed batch: the clocks need ~50 ms of load to settle
BATCHES = 5
MIN_REPS = 100


def settle(torch, step, warmup, min_ms=SETTLE_MS):
    """At least `warmup` launches and at least `min_ms` of back-to-back launches; returns the ms spent."""
    t0 = time.perf_counter()
    i = 0
    while True:
        for _ in range(20):
            step(i)
            i += 1
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3
        if ms >= min_ms and i >= warmup:
            return ms


def timed(torch, timer, step, reps):
    """Median over BATCHES batches of `reps` launches: (event ms per launch, wall ms per launch, all batches)."""
    ev, wall = [], []
    for _ in range(BATCHES):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev.append(timer.time_ms(step, reps))
        torch.cuda.synchronize()
        wall.append((time.perf_counter() - t0) * 1e3 / reps)
    return median(ev), median(wall), ev


def host_bits(t):
    import numpy as np
    return t.detach().cpu().contiguous().view(torch_int16()).numpy().view(np.uint16)


def torch_int16():
    import torch
    return torch.int16


TOL = {DT_F16: 2e-3, DT_BF16: 1e-2}   # max-abs bar of the benchmark definition per storage type


def error_stats(got_bits, ref32, ref_layer_bits, dt):
    """Distance of an output (storage bits) to the two oracles: max-abs against the fp32 oracle (the bar) and
    against the layer-style oracle (the reference CPU layer's rounding chain, src/llama2_layer_cpu.cpp:
    212-219, 675, 272-280), plus how many elements per million sit beyond the bar AND beyond two / three
    representable steps of the layer-style value."""
    import numpy as np
    from oracle import oracle as orc
    got = orc.widen(got_bits, dt)
    lay = orc.widen(ref_layer_bits, dt)
    d = np.abs(got - lay)
    mant = 7 if dt == DT_BF16 else 10
    step = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(lay.astype(np.float64)), 2.0 ** -14))) - mant)
    beyond = lambda k: float(np.count_nonzero((d > TOL[dt]) & (d > (k + 1e-4) * step))) * 1e6 / d.size
    return {"max_abs_err": float(np.abs(got - ref32).max()), "max_abs_err_layer": float(d.max()),
            "ppm_beyond_2_steps_of_layer": beyond(2), "ppm_beyond_3_steps_of_layer": beyond(3),
            "elements_checked": int(d.size)}


def merge_stats(stats):
    n = sum(s["elements_checked"] for s in stats)
    return {"max_abs_err": max(s["max_abs_err"] for s in stats),
            "max_abs_err_layer": max(s["max_abs_err_layer"] for s in stats),
            "ppm_beyond_2_steps_of_layer": sum(s["ppm_beyond_2_steps_of_layer"] * s["elements_checked"] for s in stats) / n,
            "ppm_beyond_3_steps_of_layer": sum(s["ppm_beyond_3_steps_of_layer"] * s["elements_checked"] for s in stats) / n,
            "elements_checked": n}


def bench_prefill(ops, torch, timer, S, steps, warmup, H=28, Hkv=4, clock=False, bops=None, dt=DT_BF16):
    tdt = torch.bfloat16 if dt == DT_BF16 else torch.float16
    g = torch.Generator(device="cuda").manual_seed(1004 + S)
    q = torch.randn(S, H, 128, device="cuda", dtype=torch.float32, generator=g).to(tdt)
    k = torch.randn(S, Hkv, 128, device="cuda", dtype=torch.float32, generator=g).to(tdt)
    v = torch.randn(S, Hkv, 128, device="cuda", dtype=torch.float32, generator=g).to(tdt)
    out = torch.empty_like(q)

    def step(_):
        ops.hip_flash_attn_gqa_layer(out, q, k, v, S, S, 0, H // Hkv, Hkv, 128, dt)

    settle_ms = settle(torch, step, warmup)
    reps = max(steps, MIN_REPS)
    ev_ms, wall_ms, batches = timed(torch, timer, step, reps)
    flops = 4.0 * H * 128 * S * (S + 1) / 2
    r = {"S": S, "ms_event": ev_ms, "ms_wall": wall_ms, "flops": flops, "settle_ms": settle_ms,
         "launches_per_batch": reps, "batches_us": [b * 1e3 for b in batches],
         "tflops": flops / (ev_ms * 1e-3) / 1e12}
    if clock:
        # shader clock of the first (heaviest) workgroup of one more launch, read inside the kernel
        probe = torch.zeros(2, dtype=torch.int64, device="cuda")
        for _ in range(20):
            step(0)
        bops.hip_flash_attn_gqa_clocked_layer(out, q, k, v, S, S, 0, H // Hkv, Hkv, 128, dt, probe)
        torch.cuda.synchronize()
        ticks, ref = (int(x) for x in probe.cpu())
        if ref > 0:
            r["shader_clock_mhz"] = ticks / ref * 100.0  # the reference counter runs at 100 MHz
    # accuracy of the timed output: sampled rows against the fp32 oracle (row r of a causal prefill ==
    # a one-row decode over keys 0..r)
    import numpy as np
    from oracle import oracle as orc
    qb, kb, vb, ob = (host_bits(t) for t in (q, k, v, out))
    rows = sorted(set([0, 1, 63, 64, 255, 256, S // 2, S - 1] + [int(x) for x in
                                                               np.random.default_rng(S).integers(0, S, 16)]))
    stats = []
    for row in rows:
        ref = orc.attention_f32(qb[row:row + 1], kb, vb, row + 1, row, dt)
        lay = orc.attention_layer(qb[row:row + 1], kb, vb, row + 1, row, dt)
        stats.append(error_stats(ob[row:row + 1], ref, lay, dt))
    r.update(merge_stats(stats))
    r["rows_checked"] = len(rows)
    return r, (q, k, v, out)


def bench_chunked_prefill(ops, torch, timer, m, n, steps, warmup, H=28, Hkv=4):
    """A chunk of m new tokens over a cache of n keys (offset = n - m): the prefill kernel with its key range
    split over workgroups plus the combine launch."""
    import numpy as np
    from oracle import oracle as orc
    g = torch.Generator(device="cuda").manual_seed(1004 + m + n)
    q = torch.randn(m, H, 128, device="cuda", dtype=torch.float32, generator=g).to(torch.bfloat16)
    k = torch.randn(n, Hkv, 128, device="cuda", dtype=torch.float32, generator=g).to(torch.bfloat16)
    v = torch.randn(n, Hkv, 128, device="cuda", dtype=torch.float32, generator=g).to(torch.bfloat16)
    out = torch.empty_like(q)

    def step(_):
        ops.hip_flash_attn_gqa_layer(out, q, k, v, m, n, n - m, H // Hkv, Hkv, 128, DT_BF16)

    settle(torch, step, warmup)
    ev_ms, _, _ = timed(torch, timer, step, max(steps, MIN_REPS))
    flops = 4.0 * H * 128 * (m * (n - m) + m * (m + 1) / 2)
    qb, kb, vb, ob = (host_bits(t) for t in (q, k, v, out))
    worst = 0.0
    for row in sorted({0, m // 2, m - 1}):
        ref = orc.attention_f32(qb[row:row + 1], kb, vb, n - m + row + 1, n - m + row, DT_BF16)
        worst = max(worst, float(np.abs(orc.widen(ob[row:row + 1], DT_BF16) - ref).max()))
    return {"m": m, "n": n, "H": H, "Hkv": Hkv, "us": ev_ms * 1e3, "tflops": flops / (ev_ms * 1e-3) / 1e12,
            "traffic": MEASURED_TRAFFIC_BYTES.get(("chunked", m, n)), "traffic_source": TRAFFIC_SOURCE,
            "kv_gbs": 2.0 * n * Hkv * 256 / (ev_ms * 1e-3) / 1e9, "max_abs_err": worst}


def bench_decode(ops, bops, torch, timer, batch, n, steps, warmup, H=40, Hkv=8):
    """Cold numbers: successive launches walk over distinct KV buffers whose total
    exceeds 1 GiB, so no launch is served from the 256 MB last-level cache."""
    kv_bytes = 2 * batch * n * Hkv * 128 * 2
    nbuf = max(2, -(-(1 << 30) // kv_bytes) + 1)
    g = torch.Generator(device="cuda").manual_seed(1005)
    ks, vs = [], []
    for _ in range(nbuf):
        ks.append(torch.randn(batch, n, Hkv, 128, device="cuda", dtype=torch.bfloat16, generator=g))
        vs.append(torch.randn(batch, n, Hkv, 128, device="cuda", dtype=torch.bfloat16, generator=g))
    q = torch.randn(batch, 1, H, 128, device="cuda", dtype=torch.bfloat16, generator=g)
    out = torch.empty_like(q)
    splits = ops.flash_decode_default_splits(batch, n, Hkv)
    ws_bytes = ops.flash_decode_workspace_bytes(batch, H // Hkv, Hkv, 128, splits)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")

    def step(i):
        j = i % nbuf
        ops.hip_flash_decode_gqa_layer(out, q, ks[j], vs[j], ws, ws_bytes, batch, n, n, H // Hkv,
                                       Hkv, 128, splits, DT_BF16)

    def hot(_):
        ops.hip_flash_decode_gqa_layer(out, q, ks[0], vs[0], ws, ws_bytes, batch, n, n, H // Hkv,
                                       Hkv, 128, splits, DT_BF16)

    settle(torch, step, warmup)
    reps = max(steps, MIN_REPS)
    cold, _, _ = timed(torch, timer, step, reps)
    hot_ms, _, _ = timed(torch, timer, hot, reps)
    # a kernel that only reads the same K and V arrays, cold like `step`: what the memory system delivers at
    # this byte count (the better of its two launch shapes)
    sink = torch.empty(bops.STREAM_READ_SINK_BYTES, dtype=torch.uint8, device="cuda")
    read_ms = min(timed(torch, timer, lambda i, var=var: bops.probe_stream_read(ks[i % nbuf], vs[i % nbuf], sink, var),
                        reps)[0] for var in (0, 1))
    torch.cuda.synchronize()
    # accuracy of the last timed (hot) launch: sequence 0 and the last one against the fp32 oracle
    import numpy as np
    from oracle import oracle as orc
    ob, qb = host_bits(out), host_bits(q)
    stats = []
    for b in sorted({0, batch - 1}):
        kb, vb = host_bits(ks[0][b]), host_bits(vs[0][b])
        stats.append(error_stats(ob[b], orc.attention_f32(qb[b], kb, vb, n, n - 1, DT_BF16),
                                 orc.attention_layer(qb[b], kb, vb, n, n - 1, DT_BF16), DT_BF16))
    r = {"batch": batch, "n": n, "splits": splits, "kv_bytes": kv_bytes, "buffers": nbuf,
         "ms_cold": cold, "ms_hot": hot_ms, "gbs_cold": kv_bytes / (cold * 1e-3) / 1e9,
         "gbs_hot": kv_bytes / (hot_ms * 1e-3) / 1e9,
         "ms_plain_read": read_ms, "gbs_plain_read": kv_bytes / (read_ms * 1e-3) / 1e9}
    r.update(merge_stats(stats))
    return r


def bench_decode_step(ops, torch, timer, n, steps, warmup, H=40, Hkv=8):
    """What one layer does per generated token (src/llama2_layer_npu.cpp:780-869, batch 1): the new token's
    q and k rotated, k and v appended at row n-1, attention of the one query row over the n cache rows --
    the fused rope + append launch and the reference-signature attention call (split-KV decode + combine),
    and the same step with rope and append inside the decode kernel (llmhip_decode_step_gqa)."""
    import numpy as np
    g = torch.Generator(device="cuda").manual_seed(1005 + n)
    bf = torch.bfloat16
    nbuf = max(2, -(-(1 << 30) // (2 * n * Hkv * 256)) + 1)
    kcs = [torch.randn(n, Hkv, 128, device="cuda", dtype=bf, generator=g) for _ in range(nbuf)]
    vcs = [torch.randn(n, Hkv, 128, device="cuda", dtype=bf, generator=g) for _ in range(nbuf)]
    q = torch.randn(1, H, 128, device="cuda", dtype=bf, generator=g)
    k = torch.randn(1, Hkv, 128, device="cuda", dtype=bf, generator=g)
    v = torch.randn(1, Hkv, 128, device="cuda", dtype=bf, generator=g)
    qe, out = torch.empty_like(q), torch.empty_like(q)
    table = torch.from_numpy(np.ascontiguousarray(ops.init_freq_cis(128, n, 1e6, DT_BF16))).cuda()

    def step(i):
        j = i % nbuf
        ops.hip_rope_kv_append_layer(qe, kcs[j], vcs[j], table, q, k, v, n - 1, 1, H, Hkv, 128, True, DT_BF16)
        ops.hip_flash_attn_gqa_layer(out, qe, kcs[j], vcs[j], 1, n, n - 1, H // Hkv, Hkv, 128, DT_BF16)

    def fused(i):
        j = i % nbuf
        ops.hip_decode_step_gqa_layer(out, kcs[j], vcs[j], table, q, k, v, n - 1, H // Hkv, Hkv, 128, True, DT_BF16)

    settle(torch, step, warmup)
    ms, _, _ = timed(torch, timer, step, max(steps, MIN_REPS))
    want = host_bits(out).copy()
    ms_f, _, _ = timed(torch, timer, fused, max(steps, MIN_REPS))
    same = bool((host_bits(out) == want).all())  # both paths left the result of the same buffer in `out`
    return {"n": n, "H": H, "Hkv": Hkv, "us_three_launches": ms * 1e3, "us_fused": ms_f * 1e3,
            "fused_output_bit_identical": same, "kv_gbs_fused": 2.0 * n * Hkv * 256 / (ms_f * 1e-3) / 1e9}


def bench_rope_append(ops, torch, timer, S, steps, warmup, H=28, Hkv=4):
    import numpy as np
    g = torch.Generator(device="cuda").manual_seed(7)
    q = torch.randn(S, H, 128, device="cuda", dtype=torch.bfloat16, generator=g)
    k = torch.randn(S, Hkv, 128, device="cuda", dtype=torch.bfloat16, generator=g)
    v = torch.randn(S, Hkv, 128, device="cuda", dtype=torch.bfloat16, generator=g)
    oq = torch.empty_like(q)
    kc = torch.empty(S, Hkv, 128, device="cuda", dtype=torch.bfloat16)
    vc = torch.empty_like(kc)
    table = torch.from_numpy(np.ascontiguousarray(ops.init_freq_cis(128, S, 1e6, DT_BF16))).cuda()

    def step(_):
        ops.hip_rope_kv_append_layer(oq, kc, vc, table, q, k, v, 0, S, H, Hkv, 128, True, DT_BF16)

    settle(torch, step, warmup)
    reps = max(steps, MIN_REPS)
    ms, _, _ = timed(torch, timer, step, reps)
    nbytes = 2 * S * 128 * (2 * H + 4 * Hkv) + S * 64 * 8
    # The buffers of one call (75 MB here) fit the 256 MB last-level cache, which is also how a layer
    # runs -- q, k, v were just written by the projection.  A second figure walks over enough buffer
    # sets that every call reads from and writes to HBM.
    nset = max(2, -(-(768 << 20) // nbytes))
    sets = [(torch.randn_like(q), torch.randn_like(k), torch.randn_like(v), torch.empty_like(q),
             torch.empty_like(kc), torch.empty_like(kc)) for _ in range(nset)]

    def cold(i):
        a, b, c, d, e, f = sets[i % nset]
        ops.hip_rope_kv_append_layer(d, e, f, table, a, b, c, 0, S, H, Hkv, 128, True, DT_BF16)

    cold_ms, _, _ = timed(torch, timer, cold, reps)
    # device-to-device copies that move the same number of bytes (half read, half written), timed the same way
    src = [torch.empty(nbytes // 2, dtype=torch.uint8, device="cuda") for _ in range(nset)]
    dst = [torch.empty(nbytes // 2, dtype=torch.uint8, device="cuda") for _ in range(nset)]
    copy_ms, _, _ = timed(torch, timer, lambda _: dst[0].copy_(src[0]), reps)
    copy_cold_ms, _, _ = timed(torch, timer, lambda i: dst[i % nset].copy_(src[i % nset]), reps)
    del sets, src, dst
    # bit-exact against the oracle on the first and last 32 tokens
    from oracle import oracle as orc
    tab = table.cpu().numpy()
    bad = 0
    for lo in (0, S - 32):
        sl = slice(lo, lo + 32)
        bad += int(np.count_nonzero(host_bits(oq[sl]) != orc.rope(host_bits(q[sl]), tab, lo, True, DT_BF16)))
        bad += int(np.count_nonzero(host_bits(kc[sl]) != orc.rope(host_bits(k[sl]), tab, lo, True, DT_BF16)))
        bad += int(np.count_nonzero(host_bits(vc[sl]) != host_bits(v[sl])))
    return {"S": S, "ms": ms, "bytes": nbytes, "gbs": nbytes / (ms * 1e-3) / 1e9, "mismatched_elements": bad,
            "ms_plain_copy": copy_ms, "gbs_plain_copy": nbytes / (copy_ms * 1e-3) / 1e9,
            "ms_cold": cold_ms, "gbs_cold": nbytes / (cold_ms * 1e-3) / 1e9,
            "ms_plain_copy_cold": copy_cold_ms, "gbs_plain_copy_cold": nbytes / (copy_cold_ms * 1e-3) / 1e9}


def _normal(torch, g, shape, tdt, scale=1.0):
    return (torch.randn(*shape, device="cuda", dtype=torch.float32, generator=g) * scale).to(tdt)


def bench_config1(ops, torch, timer, steps, warmup):
    """Benchmark configuration 1, Llama2-7B prefill: fp16, 32 heads = 32 kv heads, 256 tokens, theta 1e4,
    interleaved pairs.  Timed: the attention call alone (the Llama call, src/llama2_layer_npu.cpp:370-374) and
    the whole path rope -> append -> attention (fused rope + append launch, then attention)."""
    import numpy as np
    from oracle import oracle as orc
    dt, H, S = DT_F16, 32, 256
    g = torch.Generator(device="cuda").manual_seed(1001)
    q, k, v = (_normal(torch, g, (S, H, 128), torch.float16) for _ in range(3))
    qe, out = torch.empty_like(q), torch.empty_like(q)
    kc, vc = torch.zeros(512, H, 128, device="cuda", dtype=torch.float16), torch.zeros(512, H, 128, device="cuda", dtype=torch.float16)
    tab_h = ops.init_freq_cis(128, 512, 1e4, dt)
    table = torch.from_numpy(np.ascontiguousarray(tab_h)).cuda()

    def path(_):
        ops.hip_rope_kv_append_layer(qe, kc, vc, table, q, k, v, 0, S, H, H, 128, False, dt)
        ops.hip_flash_attn_opt_prefill_layer(out, qe, kc, vc, S, S, 0, H, 128, dt)

    def attn(_):
        ops.hip_flash_attn_opt_prefill_layer(out, qe, kc, vc, S, S, 0, H, 128, dt)

    settle(torch, path, warmup)
    reps = max(steps, MIN_REPS)
    us_path = timed(torch, timer, path, reps)[0] * 1e3
    us_attn = timed(torch, timer, attn, reps)[0] * 1e3
    flops = 4.0 * H * 128 * S * (S + 1) / 2
    qb, kb, vb = (host_bits(t) for t in (q, k, v))
    q_r, k_r = orc.rope(qb, tab_h, 0, False, dt), orc.rope(kb, tab_h, 0, False, dt)
    rope_bad = int(np.count_nonzero(host_bits(qe) != q_r) + np.count_nonzero(host_bits(kc[:S]) != k_r) +
                   np.count_nonzero(host_bits(vc[:S]) != vb))
    st = error_stats(host_bits(out), orc.attention_f32(q_r, k_r, vb, S, 0, dt), orc.attention_layer(q_r, k_r, vb, S, 0, dt), dt)
    r = {"config": 1, "workload": "Llama2-7B prefill: fp16, H=Hkv=32, head_dim 128, m=n=256, theta 1e4, interleaved RoPE",
         "dtype": "fp16", "flops": flops, "us_attention": us_attn, "us_rope_append_attention": us_path,
         "tflops_attention": flops / us_attn / 1e6, "tflops_path": flops / us_path / 1e6,
         "bound": "mfma", "peak_tflops": PEAK_BF16_TFLOPS, "frac": flops / us_attn / 1e6 / PEAK_BF16_TFLOPS,
         "frac_path": flops / us_path / 1e6 / PEAK_BF16_TFLOPS, "rope_append_mismatched_elements": rope_bad,
         "max_abs_err_bar": TOL[dt]}
    r.update(st)
    return r


def bench_config2(ops, torch, timer, steps, warmup):
    """Benchmark configuration 2, Llama2-7B decode step: fp16, 32 heads x 128, cache rows 0..510 filled, the new
    token rotated at position 511 and appended at row 511, attention m=1, n=512.  Timed cold (cache sets
    rotating over more than the last-level cache): the fused rope + append launch followed by the
    reference-signature attention call (decode kernel + combine), and the one-pass fused decode step."""
    import numpy as np
    from oracle import oracle as orc
    dt, H, n = DT_F16, 32, 512
    g = torch.Generator(device="cuda").manual_seed(1002)
    kv_bytes = 2 * n * H * 256
    nbuf = -(-(1 << 30) // kv_bytes) + 1
    kcs = [_normal(torch, g, (n, H, 128), torch.float16) for _ in range(nbuf)]
    vcs = [_normal(torch, g, (n, H, 128), torch.float16) for _ in range(nbuf)]
    q, k, v = (_normal(torch, g, (1, H, 128), torch.float16) for _ in range(3))
    qe, out, out_f = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    tab_h = ops.init_freq_cis(128, n, 1e4, dt)
    table = torch.from_numpy(np.ascontiguousarray(tab_h)).cuda()

    def step(i):
        j = i % nbuf
        ops.hip_rope_kv_append_layer(qe, kcs[j], vcs[j], table, q, k, v, n - 1, 1, H, H, 128, False, dt)
        ops.hip_flash_attn_opt_prefill_layer(out, qe, kcs[j], vcs[j], 1, n, n - 1, H, 128, dt)

    def fused(i):
        j = i % nbuf
        ops.hip_decode_step_gqa_layer(out_f, kcs[j], vcs[j], table, q, k, v, n - 1, 1, H, 128, False, dt)

    settle(torch, step, warmup)
    reps = max(steps, MIN_REPS) * 2
    us3 = timed(torch, timer, step, reps)[0] * 1e3
    usf = timed(torch, timer, fused, reps)[0] * 1e3
    us_hot = timed(torch, timer, lambda _: fused(0), reps)[0] * 1e3
    step(0)
    fused(0)
    torch.cuda.synchronize()
    same = bool((host_bits(out) == host_bits(out_f)).all())
    kb, vb = host_bits(kcs[0]).copy(), host_bits(vcs[0]).copy()     # row 511 now holds the appended token
    q_r = orc.rope(host_bits(q), tab_h, n - 1, False, dt)
    k_r = orc.rope(host_bits(k), tab_h, n - 1, False, dt)
    append_ok = bool((kb[n - 1] == k_r[0]).all() and (vb[n - 1] == host_bits(v)[0]).all())
    st = error_stats(host_bits(out_f), orc.attention_f32(q_r, kb, vb, n, n - 1, dt), orc.attention_layer(q_r, kb, vb, n, n - 1, dt), dt)
    r = {"config": 2, "workload": "Llama2-7B decode step: fp16, H=Hkv=32, head_dim 128, m=1, n=512 (append at row 511), "
                                  "theta 1e4, interleaved RoPE", "dtype": "fp16", "kv_bytes": kv_bytes,
         "us_three_launches_cold": us3, "us_fused_step_cold": usf, "us_fused_step_hot": us_hot,
         "gbs": kv_bytes / usf / 1e3, "bound": "hbm", "peak_gbs": PEAK_HBM_GBS, "frac": kv_bytes / usf / 1e3 / PEAK_HBM_GBS,
         "fused_equals_three_launches": same, "appended_row_bit_exact": append_ok, "max_abs_err_bar": TOL[dt],
         "note": "8 MiB of K+V per step: the step is bound by launch and memory latency, not by bandwidth"}
    r.update(st)
    return r


def bench_config3(ops, torch, timer, steps, warmup):
    """Benchmark configuration 3, Qwen2.5-1.5B: bf16, 12 heads, 2 kv heads, theta 1e6 (table rounded to bf16), neox
    pairs, q/k/v = round(x + bias) with bias ~ N(0, 0.02) as the projection leaves them.  Prefill of 256 tokens
    (rope + append, attention), then 256 decode steps with the cache growing 256 -> 512 in place, one fused
    decode-step call per token, issued back to back as a model's decode loop does; every step's output is kept
    and checked.  The same loop is also driven through the C++ layer (Qwen2AttentionLayer::Forward per token)."""
    import numpy as np
    from oracle import oracle as orc
    dt, H, Hkv, P, G = DT_BF16, 12, 2, 256, 256
    bf = torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(1003)

    def biased(rows, heads):
        x = torch.randn(rows, heads, 128, device="cuda", dtype=torch.float32, generator=g).to(bf).float()
        b = torch.randn(heads, 128, device="cuda", dtype=torch.float32, generator=g) * 0.02
        return (x + b).to(bf)

    q, k, v = biased(P + G, H), biased(P + G, Hkv), biased(P + G, Hkv)
    qe, out_p = torch.empty(P, H, 128, device="cuda", dtype=bf), torch.empty(P, H, 128, device="cuda", dtype=bf)
    outs = torch.empty(G, H, 128, device="cuda", dtype=bf)
    kc, vc = torch.zeros(P + G, Hkv, 128, device="cuda", dtype=bf), torch.zeros(P + G, Hkv, 128, device="cuda", dtype=bf)
    tab_h = ops.init_freq_cis(128, P + G, 1e6, dt)
    table = torch.from_numpy(np.ascontiguousarray(tab_h)).cuda()

    def prefill(_):
        ops.hip_rope_kv_append_layer(qe, kc, vc, table, q[:P], k[:P], v[:P], 0, P, H, Hkv, 128, True, dt)
        ops.hip_flash_attn_gqa_layer(out_p, qe, kc, vc, P, P, 0, H // Hkv, Hkv, 128, dt)

    def attn_only(_):
        ops.hip_flash_attn_gqa_layer(out_p, qe, kc, vc, P, P, 0, H // Hkv, Hkv, 128, dt)

    qs, ks_, vs_ = [q[P + i:P + i + 1] for i in range(G)], [k[P + i:P + i + 1] for i in range(G)], \
        [v[P + i:P + i + 1] for i in range(G)]
    os_ = [outs[i:i + 1] for i in range(G)]

    def decode_loop(_):
        for i in range(G):
            ops.hip_decode_step_gqa_layer(os_[i], kc, vc, table, qs[i], ks_[i], vs_[i], P + i, H // Hkv, Hkv, 128, True, dt)

    settle(torch, prefill, warmup)
    reps = max(steps, MIN_REPS)
    us_prefill = timed(torch, timer, prefill, reps)[0] * 1e3
    us_attn = timed(torch, timer, attn_only, reps)[0] * 1e3
    settle(torch, decode_loop, 1)
    loop_ms, loop_wall_ms, _ = timed(torch, timer, decode_loop, 3)
    per_step = {}
    for pos in (P, P + G // 2, P + G - 1):     # one step repeated: cache length 257, 385, 512
        i = pos - P
        per_step[str(pos + 1)] = timed(torch, timer, lambda _: ops.hip_decode_step_gqa_layer(
            os_[i], kc, vc, table, qs[i], ks_[i], vs_[i], pos, H // Hkv, Hkv, 128, True, dt), reps)[0] * 1e3
    prefill(0)
    decode_loop(0)
    torch.cuda.synchronize()
    # every step against both oracles, the caches bit for bit
    qb, kb, vb = host_bits(q), host_bits(k), host_bits(v)
    q_r = np.concatenate([orc.rope(qb[:P], tab_h, 0, True, dt)] + [orc.rope(qb[P + i:P + i + 1], tab_h, P + i, True, dt) for i in range(G)])
    k_r = np.concatenate([orc.rope(kb[:P], tab_h, 0, True, dt)] + [orc.rope(kb[P + i:P + i + 1], tab_h, P + i, True, dt) for i in range(G)])
    caches_ok = bool((host_bits(kc) == k_r).all() and (host_bits(vc) == vb).all())
    st_p = error_stats(host_bits(out_p), orc.attention_f32(q_r[:P], k_r, vb, P, 0, dt), orc.attention_layer(q_r[:P], k_r, vb, P, 0, dt), dt)
    ob = host_bits(outs)
    st_d = [error_stats(ob[i:i + 1], orc.attention_f32(q_r[P + i:P + i + 1], k_r, vb, P + i + 1, P + i, dt),
                        orc.attention_layer(q_r[P + i:P + i + 1], k_r, vb, P + i + 1, P + i, dt), dt) for i in range(G)]
    flops = 4.0 * H * 128 * P * (P + 1) / 2
    kv_bytes_total = sum(2 * (P + i + 1) * Hkv * 256 for i in range(G))
    r = {"config": 3, "workload": "Qwen2.5-1.5B: bf16, H=12, Hkv=2, head_dim 128, theta 1e6, neox RoPE, QKV bias N(0,0.02); "
                                  "prefill 256, then 256 decode steps with the cache growing 256 -> 512",
         "dtype": "bf16",
         "prefill": {"flops": flops, "us_attention": us_attn, "us_rope_append_attention": us_prefill,
                     "tflops_attention": flops / us_attn / 1e6, "bound": "mfma", "peak_tflops": PEAK_BF16_TFLOPS,
                     "frac": flops / us_attn / 1e6 / PEAK_BF16_TFLOPS, **st_p},
         "decode": {"steps": G, "us_total": loop_ms * 1e3, "us_per_token": loop_ms * 1e3 / G,
                    "host_us_per_token": loop_wall_ms * 1e3 / G,
                    "us_single_step_at_kv_length": per_step, "kv_bytes_total": kv_bytes_total,
                    "gbs": kv_bytes_total / (loop_ms * 1e-3) / 1e9, "bound": "hbm", "peak_gbs": PEAK_HBM_GBS,
                    "frac": kv_bytes_total / (loop_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                    "per_step_max_abs_err": {"max": max(x["max_abs_err"] for x in st_d),
                                             "mean": float(np.mean([x["max_abs_err"] for x in st_d]))},
                    **merge_stats(st_d),
                    "note": "0.26-0.5 MiB of K+V per step on 2 kv heads: launch-bound"},
         "caches_bit_exact": caches_ok, "max_abs_err_bar": TOL[dt],
         "frac": flops / us_attn / 1e6 / PEAK_BF16_TFLOPS,
         "reference_whole_model_context": "the reference publishes only whole-model latencies for this model and workload: "
                                          "461 ms to first token, 142 ms per token on an Orange Pi 20T (readme.md:24)"}
    return r


def layer_decode_loop(H=12, Hkv=2, prompt=256, gen=256):
    """Configuration 3's decode loop driven through the C++ device layer (Qwen2AttentionLayer::Forward per
    token: pooled tensors, no host wait per call) by the op-test binary, beside the same loop of bare C-ABI calls."""
    import subprocess
    exe = os.path.join(ROOT, "tests", "cpp", "bin", "op_test_attention_layer")
    if not os.path.exists(exe):
        return {"error": "tests/cpp/bin/op_test_attention_layer is not built"}
    r = subprocess.run([exe, "--head_num", str(H), "--kv_head_num", str(Hkv), "--prompt", str(prompt), "--steps", str(gen),
                        "--time", "5", "--dtype", "bf16", "--max_seq_len", str(prompt + gen)],
                       capture_output=True, text=True, timeout=120)
    if r.returncode != 0:
        return {"error": (r.stdout + r.stderr)[-400:]}
    return json.loads(r.stdout.strip().splitlines()[-1])


def bench_attention_block(ops, torch, timer, S, steps, warmup, H=28, Hkv=4):
    """The whole attention block of one Qwen2.5-7B layer (src/llama2_layer_npu.cpp:760-901):
    q/k/v projections with fp32 bias (hipBLASLt), fused RoPE + KV append, causal attention, o_proj,
    residual add -- random weights of that shape, one sequence of S tokens."""
    import numpy as np
    hidden, kvd = H * 128, Hkv * 128
    g = torch.Generator(device="cuda").manual_seed(11)
    bf = torch.bfloat16

    def rnd(*shape, scale=1.0):
        return (torch.randn(*shape, device="cuda", dtype=torch.float32, generator=g) * scale).to(bf)

    x, res = rnd(S, hidden), rnd(S, hidden)
    wq, wo = rnd(hidden, hidden, scale=hidden ** -0.5), rnd(hidden, hidden, scale=hidden ** -0.5)
    wk, wv = rnd(kvd, hidden, scale=hidden ** -0.5), rnd(kvd, hidden, scale=hidden ** -0.5)
    bq = torch.randn(hidden, device="cuda", generator=g) * 0.02
    bk = torch.randn(kvd, device="cuda", generator=g) * 0.02
    bv = torch.randn(kvd, device="cuda", generator=g) * 0.02
    q, k, v = torch.empty(S, hidden, device="cuda", dtype=bf), torch.empty(S, kvd, device="cuda", dtype=bf), \
        torch.empty(S, kvd, device="cuda", dtype=bf)
    qe, attn, proj, out = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    kc, vc = torch.empty(S, kvd, device="cuda", dtype=bf), torch.empty(S, kvd, device="cuda", dtype=bf)
    table = torch.from_numpy(np.ascontiguousarray(ops.init_freq_cis(128, S, 1e6, DT_BF16))).cuda()

    def proj_qkv(_):
        ops.hip_matmul_bias_layer(q, x, wq, bq, S, hidden, hidden, DT_BF16)
        ops.hip_matmul_bias_layer(k, x, wk, bk, S, kvd, hidden, DT_BF16)
        ops.hip_matmul_bias_layer(v, x, wv, bv, S, kvd, hidden, DT_BF16)

    def core(_):
        ops.hip_rope_kv_append_layer(qe, kc, vc, table, q, k, v, 0, S, H, Hkv, 128, True, DT_BF16)
        ops.hip_flash_attn_gqa_layer(attn, qe, kc, vc, S, S, 0, H // Hkv, Hkv, 128, DT_BF16)

    def tail(_):
        ops.hip_matmul_layer(proj, attn, wo, S, hidden, hidden, DT_BF16)
        ops.hip_add_layer(out, res, proj, S * hidden, DT_BF16)

    def whole(i):
        proj_qkv(i)
        core(i)
        tail(i)

    settle(torch, whole, warmup)
    r = {"S": S}
    for name, fn in (("us_total", whole), ("us_qkv_proj", proj_qkv), ("us_rope_attention", core),
                     ("us_o_proj_add", tail)):
        r[name] = timed(torch, timer, fn, max(steps, 30))[0] * 1e3
    gemm_flops = 2.0 * S * hidden * (2 * hidden + 2 * kvd)
    r["gemm_tflops"] = gemm_flops / ((r["us_qkv_proj"] + r["us_o_proj_add"]) * 1e-6) / 1e12
    return r


def cpu_baseline(S, H=28, Hkv=4):
    """The oracle's layer-style attention (the port of the reference CPU layer
    path) on the whole prefill workload: single thread (the reference's Eigen
    expressions are single-threaded) and all cores."""
    import numpy as np
    from oracle import oracle as orc
    rng = np.random.default_rng(1004 + S)
    q = orc.round_to(rng.standard_normal((S, H, 128), dtype=np.float32), DT_BF16)
    k = orc.round_to(rng.standard_normal((S, Hkv, 128), dtype=np.float32), DT_BF16)
    v = orc.round_to(rng.standard_normal((S, Hkv, 128), dtype=np.float32), DT_BF16)
    flops = 4.0 * H * 128 * S * (S + 1) / 2
    cores = min(orc.max_threads(), 16)  # the box's CPU share for one GPU is 16 threads
    t = time.perf_counter()
    orc.attention_layer(q, k, v, S, 0, DT_BF16, n_threads=cores)
    t_all = time.perf_counter() - t
    t = time.perf_counter()
    orc.attention_layer(q, k, v, S, 0, DT_BF16, n_threads=1)
    t_one = time.perf_counter() - t
    return {"value": flops / t_all / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"whole prefill workload (S={S}, H={H}, Hkv={Hkv}, bf16, {flops / 1e9:.1f} GFLOP), "
                      f"layer-style oracle: {t_all:.2f} s on {cores} threads, {t_one:.2f} s on 1 thread",
            "host_cores_visible": os.cpu_count(),
            "single_thread_value": flops / t_one / 1e12, "seconds_all_cores": t_all,
            "seconds_single_thread": t_one}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=300)
    ap.add_argument("--seq", type=int, default=4096, help="prefill sequence length of the timed step")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="", help="comma list of legs: ceiling,prefill,chunked,decode,decode_step,rope,block,configs (default all)")
    ap.add_argument("--decode-shapes", default="16x32768,1x32768,1x4096,1x16384,16x4096,16x16384",
                    help="comma list of BATCHxKVLEN decode cases; the first one is the headline")
    ap.add_argument("--chunk-shapes", default="256x33024x28x4,40x131072x40x8",
                    help="comma list of MxNxHxHKV chunked-prefill cases (M new tokens over a cache of N keys)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run a plain 1 GiB device copy a few times (known traffic: 1 GiB read + "
                         "1 GiB written per launch) so that FETCH_SIZE / WRITE_SIZE of a rocprofv3 --pmc run "
                         "can be scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build measures one GPU; --gpus must be 1 "
            "(the path shards by kv head without any exchange between GPUs)")
        sys.exit(2)

    import torch
    import llm_simple_amd.ops as ops
    import llm_simple_amd.bench_ops as bops  # the measurement library: clock stamp, MFMA ceiling, plain read
    if not torch.cuda.is_available():
        log("bench.py: no GPU visible")
        sys.exit(1)
    torch.cuda.set_device(0)
    timer = HipTimer(ops.lib)
    legs = set(args.only.split(",")) if args.only else {"ceiling", "prefill", "chunked", "decode", "decode_step", "rope", "block", "configs"}
    legs.discard("none")
    extra = {}

    cus, max_mhz, _ = ops.device_props(0)
    # dense bf16 MFMA: 4 SIMDs x 1024 flop per clock per CU (one 32x32x16 MFMA = 32768 flop in 32 cycles)
    box_peak_tflops = cus * max_mhz * 1e6 * 4096 / 1e12

    # what the matrix pipe of this box sustains on N(0,1) operands: alone, and with the other
    # instructions of an attention inner loop beside the MFMAs (no memory traffic, no barriers)
    ceiling = None
    if "ceiling" in legs:
        ceiling = {"mfma_only_tflops": bops.probe_mfma_ceiling(0, 150.0),
                   "attention_mix_tflops": bops.probe_mfma_ceiling(1, 150.0),
                   "what": "sustained bf16 32x32x16 MFMA rate on N(0,1) operands, 8 waves per CU: the MFMAs alone, "
                           "and with 6 LDS fragment reads, 13 vector instructions and 4 v_exp_f32 per 4 MFMAs "
                           "beside them (the prefill loop's mix) -- no memory traffic, barriers or dependences"}
        log(f"MFMA ceiling on N(0,1) operands: alone {ceiling['mfma_only_tflops']:.0f} TFLOP/s, "
            f"with the attention instruction mix {ceiling['attention_mix_tflops']:.0f} TFLOP/s")

    # ---- the timed step: prefill at the headline shape ----
    torch.cuda.synchronize()
    pre, _ = bench_prefill(ops, torch, timer, args.seq, args.steps, args.warmup, clock=True, bops=bops)
    log(f"prefill S={args.seq}: {pre['ms_event'] * 1e3:.1f} us  {pre['tflops']:.1f} TFLOP/s  "
        f"max-abs {pre['max_abs_err']:.2e}  shader clock {pre.get('shader_clock_mhz', 0):.0f} MHz")
    if "prefill" in legs:
        others = []
        for S in (1024, 8192):
            if S == args.seq:
                continue
            r, _ = bench_prefill(ops, torch, timer, S, args.steps, args.warmup)
            log(f"prefill S={S}: {r['ms_event'] * 1e3:.1f} us  {r['tflops']:.1f} TFLOP/s  max-abs {r['max_abs_err']:.2e}")
            others.append({"S": S, "us": r["ms_event"] * 1e3, "tflops": r["tflops"],
                           "frac": r["tflops"] / PEAK_BF16_TFLOPS, "max_abs_err": r["max_abs_err"],
                           "max_abs_err_layer": r["max_abs_err_layer"]})
        extra["prefill_other"] = others
        # the same kernel on fp16 (the reference's Llama models; same published peak)
        r, _ = bench_prefill(ops, torch, timer, args.seq, args.steps, args.warmup, dt=DT_F16)
        log(f"prefill fp16 S={args.seq}: {r['ms_event'] * 1e3:.1f} us  {r['tflops']:.1f} TFLOP/s  max-abs {r['max_abs_err']:.2e}")
        extra["prefill_fp16"] = {"S": args.seq, "us": r["ms_event"] * 1e3, "tflops": r["tflops"],
                                 "frac": r["tflops"] / PEAK_BF16_TFLOPS, "max_abs_err": r["max_abs_err"],
                                 "max_abs_err_layer": r["max_abs_err_layer"], "max_abs_err_bar": TOL[DT_F16]}

    if "chunked" in legs:
        rows = []
        for (m, n, H, Hkv) in [tuple(int(x) for x in c.split("x")) for c in args.chunk_shapes.split(",") if c]:
            r = bench_chunked_prefill(ops, torch, timer, m, n, args.steps, args.warmup, H, Hkv)
            log(f"chunked prefill m={m} n={n} H={H} Hkv={Hkv}: {r['us']:.1f} us  {r['tflops']:.0f} TFLOP/s  "
                f"K+V {r['kv_gbs']:.0f} GB/s  max-abs {r['max_abs_err']:.2e}")
            rows.append(r)
        extra["chunked_prefill"] = rows

    if "decode" in legs:
        dec = []
        shapes = [tuple(int(x) for x in c.split("x")) for c in args.decode_shapes.split(",") if c]
        for batch, n in shapes:
            r = bench_decode(ops, bops, torch, timer, batch, n, args.steps, args.warmup)
            log(f"decode B={batch} n={n} splits={r['splits']}: cold {r['ms_cold'] * 1e3:.1f} us "
                f"{r['gbs_cold']:.0f} GB/s, hot {r['ms_hot'] * 1e3:.1f} us {r['gbs_hot']:.0f} GB/s, "
                f"max-abs {r['max_abs_err']:.2e}; a plain read of the same arrays, cold: "
                f"{r['ms_plain_read'] * 1e3:.1f} us {r['gbs_plain_read']:.0f} GB/s")
            dec.append(r)
            torch.cuda.empty_cache()
        head = dec[0]
        extra["decode_value"] = head["gbs_cold"]
        extra["decode_unit"] = "GB/s"
        extra["roofline_decode"] = {
            "bound": "hbm", "achieved": head["gbs_cold"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": head["gbs_cold"] / PEAK_HBM_GBS,
            "traffic": MEASURED_TRAFFIC_BYTES.get(("decode", head["batch"], head["n"])),
            "traffic_source": TRAFFIC_SOURCE, "max_abs_err": head["max_abs_err"],
            "box": {"plain_read_gbs": head["gbs_plain_read"],
                    "frac_of_plain_read": head["gbs_cold"] / head["gbs_plain_read"],
                    "plain_read": "a kernel that only reads the same K and V arrays once, cold, timed the same way "
                                  "(llmhip_bench_stream_read)"},
            "workload": f"Qwen2.5-32B decode bf16 H=40 Hkv=8 n={head['n']} batch={head['batch']} "
                        f"({head['kv_bytes'] / 2 ** 20:.0f} MiB of K+V per launch, cold)"}
        extra["decode_all"] = [
            {"batch": r["batch"], "n": r["n"], "splits": r["splits"], "us_cold": r["ms_cold"] * 1e3,
             "gbs_cold": r["gbs_cold"], "frac_cold": r["gbs_cold"] / PEAK_HBM_GBS,
             "us_hot": r["ms_hot"] * 1e3, "gbs_hot": r["gbs_hot"], "max_abs_err": r["max_abs_err"],
             "max_abs_err_layer": r["max_abs_err_layer"],
             "us_plain_read": r["ms_plain_read"] * 1e3, "frac_of_plain_read": r["ms_plain_read"] / r["ms_cold"]}
            for r in dec]

    if "decode_step" in legs:
        extra["decode_step"] = [bench_decode_step(ops, torch, timer, n, args.steps, args.warmup) for n in (4096, 32768)]
        for r in extra["decode_step"]:
            log(f"decode step B=1 n={r['n']}: rope+append, decode, combine {r['us_three_launches']:.1f} us; fused into the "
                f"decode kernel {r['us_fused']:.1f} us ({r['kv_gbs_fused']:.0f} GB/s), bit-identical {r['fused_output_bit_identical']}")
        torch.cuda.empty_cache()

    if "rope" in legs:
        r = bench_rope_append(ops, torch, timer, args.seq, args.steps, args.warmup)
        log(f"rope+append S={args.seq}: buffers in the last-level cache {r['ms'] * 1e3:.1f} us {r['gbs']:.0f} GB/s, from and to "
            f"HBM {r['ms_cold'] * 1e3:.1f} us {r['gbs_cold']:.0f} GB/s; a device-to-device copy moving the same bytes: "
            f"{r['ms_plain_copy'] * 1e3:.1f} us {r['gbs_plain_copy']:.0f} GB/s and {r['ms_plain_copy_cold'] * 1e3:.1f} us "
            f"{r['gbs_plain_copy_cold']:.0f} GB/s")
        extra["rope_kv_append"] = {
            "S": r["S"],
            # from and to HBM (buffer sets rotating over more than the last-level cache): the HBM roofline figure
            "us_cold": r["ms_cold"] * 1e3, "gbs_cold": r["gbs_cold"], "frac": r["gbs_cold"] / PEAK_HBM_GBS,
            "us_plain_copy_cold": r["ms_plain_copy_cold"] * 1e3, "gbs_plain_copy_cold": r["gbs_plain_copy_cold"],
            # the same buffers every call (they fit the last-level cache, as q, k, v fresh from the projection do)
            "us_cached": r["ms"] * 1e3, "gbs_cached": r["gbs"],
            "us_plain_copy_cached": r["ms_plain_copy"] * 1e3, "gbs_plain_copy_cached": r["gbs_plain_copy"],
            "traffic": MEASURED_TRAFFIC_BYTES.get(("rope", r["S"])), "traffic_source": TRAFFIC_SOURCE,
            "mismatched_elements": r["mismatched_elements"]}

    if "block" in legs:
        r = bench_attention_block(ops, torch, timer, args.seq, args.steps // 8, 3)
        log(f"attention block S={args.seq}: {r['us_total']:.0f} us (qkv proj {r['us_qkv_proj']:.0f}, "
            f"rope+attention {r['us_rope_attention']:.0f}, o_proj+add {r['us_o_proj_add']:.0f}; "
            f"GEMMs {r['gemm_tflops']:.0f} TFLOP/s)")
        extra["attention_block"] = r

    if "configs" in legs:
        try:
            # one entry per benchmark configuration (BASELINE.json configs[0..4]); 4 and 5 summarise the legs above
            c1 = bench_config1(ops, torch, timer, args.steps, args.warmup)
            log(f"config 1 (Llama2-7B prefill fp16 S=256): attention {c1['us_attention']:.1f} us {c1['tflops_attention']:.0f} TFLOP/s, "
                f"rope+append+attention {c1['us_rope_append_attention']:.1f} us, max-abs {c1['max_abs_err']:.2e} "
                f"(layer-style {c1['max_abs_err_layer']:.2e})")
            c2 = bench_config2(ops, torch, timer, args.steps, args.warmup)
            log(f"config 2 (Llama2-7B decode fp16 n=512): three launches {c2['us_three_launches_cold']:.1f} us, fused step "
                f"{c2['us_fused_step_cold']:.1f} us ({c2['gbs']:.0f} GB/s), max-abs {c2['max_abs_err']:.2e} "
                f"(layer-style {c2['max_abs_err_layer']:.2e})")
            torch.cuda.empty_cache()
            c3 = bench_config3(ops, torch, timer, args.steps, args.warmup)
            c3["decode"]["through_cpp_layer"] = layer_decode_loop()
            lay = c3["decode"]["through_cpp_layer"]
            log(f"config 3 (Qwen2.5-1.5B bf16): prefill 256 attention {c3['prefill']['us_attention']:.1f} us, with rope+append "
                f"{c3['prefill']['us_rope_append_attention']:.1f} us; 256 decode steps {c3['decode']['us_total']:.0f} us = "
                f"{c3['decode']['us_per_token']:.2f} us/token from Python; from C++: C-ABI calls "
                f"{lay.get('abi_decode_us_per_step', float('nan')):.2f} us/token, through Qwen2AttentionLayer "
                f"{lay.get('layer_decode_us_per_step', float('nan')):.2f} us/token (host {lay.get('layer_host_us_per_step', float('nan')):.2f}); "
                f"max-abs prefill {c3['prefill']['max_abs_err']:.2e}, decode {c3['decode']['max_abs_err']:.2e}")
            cfgs = [c1, c2, c3]
            c4 = {"config": 4, "workload": "Qwen2.5-7B prefill: bf16, H=28, Hkv=4, head_dim 128, S in {1024, 4096, 8192}",
                  "dtype": "bf16", "bound": "mfma", "peak_tflops": PEAK_BF16_TFLOPS,
                  "shapes": [{"S": args.seq, "us": pre["ms_event"] * 1e3, "tflops": pre["tflops"],
                              "frac": pre["tflops"] / PEAK_BF16_TFLOPS, "max_abs_err": pre["max_abs_err"],
                              "max_abs_err_layer": pre["max_abs_err_layer"]}] + extra.get("prefill_other", []),
                  "frac": pre["tflops"] / PEAK_BF16_TFLOPS, "max_abs_err": pre["max_abs_err"],
                  "max_abs_err_layer": pre["max_abs_err_layer"], "max_abs_err_bar": TOL[DT_BF16]}
            cfgs.append(c4)
            if "decode_all" in extra:
                c5 = {"config": 5, "workload": "Qwen2.5-32B decode: bf16, H=40, Hkv=8, head_dim 128, n in {4096, 16384, 32768}, "
                                               "batch in {1, 16}, cold", "dtype": "bf16", "bound": "hbm", "peak_gbs": PEAK_HBM_GBS,
                      "shapes": extra["decode_all"], "frac": extra["roofline_decode"]["frac"],
                      "max_abs_err": max(x["max_abs_err"] for x in extra["decode_all"]),
                      "max_abs_err_layer": max(x["max_abs_err_layer"] for x in extra["decode_all"]),
                      "max_abs_err_bar": TOL[DT_BF16]}
                cfgs.append(c5)
            extra["configs"] = cfgs
        except Exception as e:  # the headline line must still be printed
            log(f"configs leg failed: {e!r}")
            extra["configs_error"] = repr(e)

    if args.calib_copy:
        src = torch.empty(1 << 29, dtype=torch.bfloat16, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        extra["calib_copy_bytes_each_way"] = src.numel() * 2
        del src, dst

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(args.seq)
        log(f"cpu baseline: {cpu['sample']}")

    line = {
        "metric": METRIC,
        "value": pre["tflops"],
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": pre["ms_wall"],
        "settle_ms": pre["settle_ms"],
        "timing": f"clock-settle phase of >= {SETTLE_MS:.0f} ms of launches, then the median of {BATCHES} batches of "
                  f"{pre['launches_per_batch']} back-to-back launches between two HIP events on the launch stream",
        "max_abs_err": pre["max_abs_err"],
        "max_abs_err_bar": 1e-2,
        "max_abs_err_layer": pre["max_abs_err_layer"],
        "layer_oracle": {"what": "distance of the same sampled rows to the layer-style oracle (scores, probabilities and "
                                 "output rounded to the storage type, src/llama2_layer_cpu.cpp:212-219, 675, 272-280), "
                                 "whose own distance to the fp32 golden exceeds the bf16 bar on rows that see few keys",
                         "ppm_beyond_2_steps": pre["ppm_beyond_2_steps_of_layer"],
                         "ppm_beyond_3_steps": pre["ppm_beyond_3_steps_of_layer"],
                         "elements_checked": pre["elements_checked"]},
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"Qwen2.5-7B causal prefill attention, bf16, batch 1, H=28, Hkv=4, "
                               f"head_dim=128, S={args.seq} (BASELINE.json configs[3]); decode leg: "
                               f"Qwen2.5-32B H=40 Hkv=8 n=32768 (BASELINE.json configs[4])"},
        "roofline": {"bound": "mfma", "achieved": pre["tflops"], "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": pre["tflops"] / PEAK_BF16_TFLOPS,
                     "traffic": MEASURED_TRAFFIC_BYTES.get(("prefill", args.seq)),
                     "traffic_source": TRAFFIC_SOURCE,
                     "kernel": "flash_prefill_kernel<bf16>", "us_per_launch": pre["ms_event"] * 1e3,
                     "batches_us": pre["batches_us"],
                     "flops_per_launch": pre["flops"],
                     "peak_source": "published MI355X dense bf16 MFMA peak (2.5 PFLOP/s, assumes 2.4 GHz)",
                     "box": {"compute_units": cus, "max_shader_clock_mhz": max_mhz,
                             "peak_at_max_clock_tflops": box_peak_tflops,
                             "shader_clock_under_load_mhz": pre.get("shader_clock_mhz"),
                             "measured_ceiling": ceiling,
                             "frac_of_attention_mix_ceiling":
                                 (pre["tflops"] / ceiling["attention_mix_tflops"]) if ceiling else None,
                             "peak_at_clock_under_load_tflops":
                                 (cus * pre["shader_clock_mhz"] * 1e6 * 4096 / 1e12)
                                 if pre.get("shader_clock_mhz") else None}},
        "cpu_baseline": cpu,
    }
    line.update(extra)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
