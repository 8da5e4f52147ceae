"""Stream behaviour of the operators through the C ABI: they run on the stream they are given (results on a
created stream equal the default-stream results bit for bit), and the launches that allocate nothing can be
captured in a HIP graph and replayed (every replay checked against the eager result, with eager work and
synchronisations between the replays)."""
import ctypes

import numpy as np
import pytest

from helpers import DT_BFLOAT16, DT_FLOAT16, dev_empty, f32_dev, normal_bits, to_dev, to_host
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def _chain(ops, stream, d_table, d_q, d_k, d_v, d_kc, d_vc, d_qe, d_o, d_q1, d_o1, m, H, Hkv, dt):
    """rope + append of m tokens at row 0, causal attention over them, then one decode step over the cache."""
    ops.hip_rope_kv_append_layer(d_qe, d_kc, d_vc, d_table, d_q, d_k, d_v, 0, m, H, Hkv, 128, True, dt, stream)
    ops.hip_flash_attn_gqa_layer(d_o, d_qe, d_kc, d_vc, m, m, 0, H // Hkv, Hkv, 128, dt, stream)
    ops.hip_flash_decode_gqa_static_layer(d_o1, d_q1, d_kc, d_vc, 1, m, m, H // Hkv, Hkv, 128, 0, dt, stream)


@pytest.mark.parametrize("dt", [DT_BFLOAT16, DT_FLOAT16])
def test_created_stream_equals_default_stream(dt):
    import torch
    import llm_simple_amd.ops as ops
    m, H, Hkv = 300, 12, 2
    table = f32_dev(orc.init_freq_cis(128, 512, 1e6, dt))
    q, k, v = (to_dev(normal_bits(s, (m, h, 128), dt)) for s, h in ((1, H), (2, Hkv), (3, Hkv)))
    q1 = to_dev(normal_bits(4, (1, H, 128), dt))
    outs = []
    s = ctypes.c_void_p()
    assert ops.lib.llmhip_stream_create(ctypes.byref(s)) == 0
    try:
        for stream in (0, s.value):
            kc, vc = dev_empty((512, Hkv, 128)).zero_(), dev_empty((512, Hkv, 128)).zero_()
            qe, o, o1 = dev_empty((m, H, 128)), dev_empty((m, H, 128)), dev_empty((1, H, 128))
            torch.cuda.synchronize()
            _chain(ops, stream, table, q, k, v, kc, vc, qe, o, q1, o1, m, H, Hkv, dt)
            # also the reference-signature decode (per-stream scratch of the library)
            o2 = dev_empty((1, H, 128))
            ops.hip_flash_attn_gqa_layer(o2, q1, kc, vc, 1, m, m - 1, H // Hkv, Hkv, 128, dt, stream)
            assert ops.lib.llmhip_stream_sync(stream) == 0
            outs.append([to_host(t).copy() for t in (qe, kc, vc, o, o1, o2)])
        for a, b in zip(*outs):
            assert np.array_equal(a, b)
        assert np.array_equal(outs[0][4], outs[0][5])  # static decode == reference-signature decode
    finally:
        assert ops.lib.llmhip_stream_destroy(s) == 0


def test_graph_capture_and_replay():
    import torch
    import llm_simple_amd.ops as ops
    dt, m, H, Hkv = DT_BFLOAT16, 200, 28, 4
    table = f32_dev(orc.init_freq_cis(128, 256, 1e6, dt))
    mk = lambda seed, h, rows=m: to_dev(normal_bits(seed, (rows, h, 128), dt))
    d_q, d_k, d_v, d_q1 = mk(10, H), mk(11, Hkv), mk(12, Hkv), mk(13, H, 1)
    kc, vc = dev_empty((256, Hkv, 128)).zero_(), dev_empty((256, Hkv, 128)).zero_()
    qe, o, o1 = dev_empty((m, H, 128)), dev_empty((m, H, 128)), dev_empty((1, H, 128))
    torch.cuda.synchronize()
    # eager once first (module load, LDS attribute of the kernels): nothing of that belongs in a capture
    _chain(ops, 0, table, d_q, d_k, d_v, kc, vc, qe, o, d_q1, o1, m, H, Hkv, dt)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _chain(ops, torch.cuda.current_stream().cuda_stream, table, d_q, d_k, d_v, kc, vc, qe, o, d_q1, o1, m, H,
               Hkv, dt)
    for rep in range(4):
        # new inputs in the captured buffers, eager result into separate outputs
        for t, seed, h, rows in ((d_q, 100, H, m), (d_k, 200, Hkv, m), (d_v, 300, Hkv, m), (d_q1, 400, H, 1)):
            t.copy_(to_dev(normal_bits(seed + rep, (rows, h, 128), dt)))
        kc2, vc2 = dev_empty((256, Hkv, 128)).zero_(), dev_empty((256, Hkv, 128)).zero_()
        qe2, o2, o12 = dev_empty((m, H, 128)), dev_empty((m, H, 128)), dev_empty((1, H, 128))
        _chain(ops, 0, table, d_q, d_k, d_v, kc2, vc2, qe2, o2, d_q1, o12, m, H, Hkv, dt)
        torch.cuda.synchronize()
        want = [to_host(t).copy() for t in (qe2, kc2, vc2, o2, o12)]
        for t in (qe, o, o1):
            t.fill_(0x7FFF)  # stale results must not survive
        kc.zero_()
        vc.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [to_host(t).copy() for t in (qe, kc, vc, o, o1)]
        for a, b in zip(got, want):
            assert np.array_equal(a, b), f"replay {rep}"


def test_scratch_does_not_grow_under_capture():
    """A reference-signature call whose per-stream scratch would have to grow while its stream is being captured
    is refused with LLMHIP_ERR_WORKSPACE (growing allocates); after the stream has been warmed up with the shape,
    the same call is captured, and replays give the eager result."""
    import torch
    import llm_simple_amd.ops as ops
    dt, H, Hkv, n = DT_BFLOAT16, 40, 8, 40000   # the default split count for this cache needs more than 4 MiB? no:
    # 8 kv heads x 32 splits x 8320 bytes = 2.1 MB fits the first 4 MiB buffer, so ask for a chunk whose partials do not
    m = 24                                        # 24 tokens over 40000 keys: key-range split, fp32 partials
    need = ops.lib.llmhip_flash_attn_scratch_bytes(m, n, n - m, H // Hkv, Hkv)
    assert need > (4 << 20), need
    q = to_dev(normal_bits(31, (m, H, 128), dt))
    k, v = (to_dev(normal_bits(s, (n, Hkv, 128), dt)) for s in (32, 33))
    o, o_small = dev_empty((m, H, 128)), dev_empty((1, H, 128))
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        sp = side.cuda_stream
        # first call on this stream: a small decode allocates the 4 MiB buffer
        ops.hip_flash_attn_gqa_layer(o_small, q[:1], k, v, 1, 4096, 4095, H // Hkv, Hkv, 128, dt, sp)
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        refused = None
        with torch.cuda.graph(graph, stream=side):
            cap = torch.cuda.current_stream().cuda_stream
            ops.hip_flash_attn_gqa_layer(o_small, q[:1], k, v, 1, 4096, 4095, H // Hkv, Hkv, 128, dt, cap)   # fits: captured
            refused = ops.lib.llmhip_flash_attn_gqa(o.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), m, n, n - m,
                                                    H // Hkv, Hkv, 128, dt, cap)
        assert refused == -3, refused
    torch.cuda.synchronize()
    # the refused call left the capture intact: the graph replays the small decode
    want = dev_empty((1, H, 128))
    ops.hip_flash_attn_gqa_layer(want, q[:1], k, v, 1, 4096, 4095, H // Hkv, Hkv, 128, dt)
    o_small.fill_(0x7FFF)
    graph.replay()
    torch.cuda.synchronize()
    assert np.array_equal(to_host(o_small), to_host(want))


def test_memset_async_fills_exactly_the_range():
    """llmhip_memset_async is a fill kernel (it may be captured into a HIP graph): any alignment, any size, nothing
    outside the range touched."""
    import torch
    import llm_simple_amd.ops as ops
    for off, n in ((0, 1 << 20), (3, 1000), (5, 7), (16, 16), (1, 4097), (9, 0), (13, (1 << 22) + 11)):
        buf = torch.full((n + 64,), 0x11, dtype=torch.uint8, device="cuda")
        assert ops.lib.llmhip_memset_async(buf.data_ptr() + off, 0xA5, n, None) == 0
        torch.cuda.synchronize()
        got = buf.cpu().numpy()
        assert (got[:off] == 0x11).all() and (got[off:off + n] == 0xA5).all() and (got[off + n:] == 0x11).all(), (off, n)


def test_measurement_aids():
    """Measurement library (libllmhip_bench.so): the clocked prefill entry returns the same output as the plain one and plausible counters; the MFMA
    ceiling probe returns a rate between a tenth of the published peak and the peak."""
    import torch
    import llm_simple_amd.bench_ops as bops
    import llm_simple_amd.ops as ops
    dt, S, H, Hkv = DT_BFLOAT16, 512, 8, 2
    q, k, v = (to_dev(normal_bits(s, (S, h, 128), dt)) for s, h in ((21, H), (22, Hkv), (23, Hkv)))
    o_a, o_b = dev_empty((S, H, 128)), dev_empty((S, H, 128))
    probe = torch.zeros(2, dtype=torch.int64, device="cuda")
    ops.hip_flash_attn_gqa_layer(o_a, q, k, v, S, S, 0, H // Hkv, Hkv, 128, dt)
    bops.hip_flash_attn_gqa_clocked_layer(o_b, q, k, v, S, S, 0, H // Hkv, Hkv, 128, dt, probe)
    torch.cuda.synchronize()
    assert np.array_equal(to_host(o_a), to_host(o_b))
    ticks, ref = (int(x) for x in probe.cpu())
    assert ticks > 0 and ref > 0 and 300.0 < ticks / ref * 100.0 < 3000.0   # MHz
    # decode-sized shapes are refused by the clocked entry (it times the prefill kernel only)
    assert bops.lib.llmhip_bench_flash_attn_gqa_clocked(o_b.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), 1, S,
                                                 S - 1, H // Hkv, Hkv, 128, dt, probe.data_ptr(), None) == -2
    alone, mix = bops.probe_mfma_ceiling(0, 5.0), bops.probe_mfma_ceiling(1, 5.0)
    assert 250.0 < mix < alone < 2600.0, (alone, mix)
    cus, mhz, mem = ops.device_props(0)
    assert cus >= 64 and 1000.0 <= mhz <= 3000.0 and mem > (16 << 30)


def test_plain_read_probe_reads_every_byte():
    """llmhip_bench_stream_read XORs everything it reads into one word per wave: the XOR of those words must be
    the XOR of all 32-bit words of both arrays, for both launch shapes and a size that is not a multiple of the
    grid's stride."""
    import torch
    import llm_simple_amd.bench_ops as bops
    rng = np.random.default_rng(5)
    for n_words in (4 * 1000, 4 * 262144 + 4 * 37):
        a = rng.integers(0, 2 ** 32, n_words, dtype=np.uint32)
        b = rng.integers(0, 2 ** 32, n_words, dtype=np.uint32)
        want = int(np.bitwise_xor.reduce(a) ^ np.bitwise_xor.reduce(b))
        d_a, d_b = to_dev(a.view(np.uint16)), to_dev(b.view(np.uint16))
        for variant in (0, 1):
            sink = torch.zeros(bops.STREAM_READ_SINK_BYTES // 4, dtype=torch.int32, device="cuda")
            bops.probe_stream_read(d_a, d_b, sink, variant)
            torch.cuda.synchronize()
            got = int(np.bitwise_xor.reduce(sink.cpu().numpy().view(np.uint32)))
            assert got == want, (n_words, variant, hex(got), hex(want))

