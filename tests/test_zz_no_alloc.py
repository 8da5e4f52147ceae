"""The allocation-free decode entry point (llmhip_flash_decode_gqa_static), through the C ABI, against
llmhip_flash_decode_gqa on the same inputs: same kernels, same split count, so the outputs must be
bit-identical.  Two calls in a row share the library's fixed scratch array, the second with a smaller
input (fewer sequences, shorter cache, fewer splits) whose result must not see the first call's
partials; plus the oracle on the second call, and the size limit."""
import ctypes

import numpy as np
import pytest

from helpers import DT_BFLOAT16, DT_FLOAT16, check_attention, dev_empty, normal_bits, to_dev, to_host

pytestmark = pytest.mark.gpu


def _both(ops, torch, q, k, v, batch, n, stride, g, Hkv, splits, dt):
    ns = splits if splits > 0 else ops.flash_decode_default_splits(batch, n, Hkv)
    wsb = ops.flash_decode_workspace_bytes(batch, g, Hkv, 128, ns)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda")
    dq, dk, dv = to_dev(q), to_dev(k), to_dev(v)
    want, got = dev_empty(q.shape), dev_empty(q.shape)
    ops.hip_flash_decode_gqa_layer(want, dq, dk, dv, ws, wsb, batch, n, stride, g, Hkv, 128, splits, dt)
    torch.cuda.synchronize()
    # "allocates nothing" is checked on the device itself (hipMemGetInfo), not in torch's caching allocator,
    # which cannot see a hipMalloc made inside the library; torch's own counters must not move either
    before_free, before_torch = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
    ops.hip_flash_decode_gqa_static_layer(got, dq, dk, dv, batch, n, stride, g, Hkv, 128, splits, dt)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == before_free and torch.cuda.memory_reserved() == before_torch
    return to_host(want), to_host(got)


def test_device_free_bytes_see_a_library_allocation():
    """The detector of the test above works: a device allocation made through the library (the size of the
    per-stream scratch that the static entry point must not touch) lowers the device's free bytes, and
    torch's counters do not notice it."""
    import torch
    import llm_simple_amd.ops as ops
    torch.cuda.synchronize()
    free0, torch0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    p = ctypes.c_void_p()
    assert ops.lib.llmhip_malloc(ctypes.byref(p), 4 << 20) == 0
    free1 = torch.cuda.mem_get_info()[0]
    assert ops.lib.llmhip_free(p) == 0
    assert free1 <= free0 - (4 << 20) and torch.cuda.memory_allocated() == torch0
    assert torch.cuda.mem_get_info()[0] == free0


@pytest.mark.parametrize("dt", [DT_BFLOAT16, DT_FLOAT16])
def test_static_decode_matches_workspace_decode_twice(dt):
    import torch
    import llm_simple_amd.ops as ops
    H, Hkv = 40, 8
    g = H // Hkv
    # first call: 3 sequences, 5000 keys (stride 5120), default split count
    b1, n1, s1 = 3, 5000, 5120
    q = normal_bits(41, (b1, 1, H, 128), dt)
    k = normal_bits(42, (b1, s1, Hkv, 128), dt)
    v = normal_bits(43, (b1, s1, Hkv, 128), dt)
    k[:, n1:] = 0x7FFF  # rows past n must not be read
    v[:, n1:] = 0x7FFF
    want, got = _both(ops, torch, q, k, v, b1, n1, s1, g, Hkv, 0, dt)
    assert np.array_equal(got, want)
    check_attention(got, q, k, v, n1, n1 - 1, dt, batch=True)
    # second call, smaller in every respect: 1 sequence, 700 keys, 3 splits
    b2, n2 = 1, 700
    q2 = normal_bits(51, (b2, 1, H, 128), dt)
    k2 = normal_bits(52, (b2, n2, Hkv, 128), dt)
    v2 = normal_bits(53, (b2, n2, Hkv, 128), dt)
    want2, got2 = _both(ops, torch, q2, k2, v2, b2, n2, n2, g, Hkv, 3, dt)
    assert np.array_equal(got2, want2)
    check_attention(got2, q2, k2, v2, n2, n2 - 1, dt, batch=True)
    # and a single split (no scratch at all)
    want3, got3 = _both(ops, torch, q2, k2, v2, b2, n2, n2, g, Hkv, 1, dt)
    assert np.array_equal(got3, want3)


def test_static_decode_rejects_what_does_not_fit():
    import llm_simple_amd.ops as ops
    lib = ops.lib
    cap = lib.llmhip_flash_decode_static_scratch_bytes()
    assert cap == 4 << 20
    buf = ctypes.create_string_buffer(96)
    p = (ctypes.addressof(buf) + 15) & ~15  # the entry points refuse misaligned pointers
    # 64 sequences x 8 kv heads x 2 splits = 1024 slots of 8320 bytes > 4 MiB: rejected before any launch
    assert ops.flash_decode_workspace_bytes(64, 5, 8, 128, 2) > cap
    assert lib.llmhip_flash_decode_gqa_static(p, p, p, p, 64, 4096, 4096, 5, 8, 128, 2, DT_BFLOAT16, None) == -3
    assert lib.llmhip_flash_decode_gqa_static(None, p, p, p, 1, 16, 16, 5, 8, 128, 1, DT_BFLOAT16, None) == -1
    assert lib.llmhip_flash_decode_gqa_static(p, p, p, p, 1, 16, 16, 5, 8, 64, 1, DT_BFLOAT16, None) == -2


def test_static_decode_lowers_a_default_split_count_that_does_not_fit():
    """40 sequences x 8 kv heads: the default rule asks for several splits, whose partials would not fit the
    fixed array; with num_splits <= 0 the call takes the largest count that fits (here one split) and must
    equal the workspace decode run with that count."""
    import torch
    import llm_simple_amd.ops as ops
    H, Hkv, batch, n, dt = 40, 8, 40, 2048, DT_BFLOAT16
    g = H // Hkv
    default = ops.flash_decode_default_splits(batch, n, Hkv)
    cap = ops.lib.llmhip_flash_decode_static_scratch_bytes()
    assert default > 1 and ops.flash_decode_workspace_bytes(batch, g, Hkv, 128, default) > cap
    fits = max(s for s in range(1, default) if ops.flash_decode_workspace_bytes(batch, g, Hkv, 128, s) <= cap)
    q = normal_bits(61, (batch, 1, H, 128), dt)
    k = normal_bits(62, (batch, n, Hkv, 128), dt)
    v = normal_bits(63, (batch, n, Hkv, 128), dt)
    dq, dk, dv = to_dev(q), to_dev(k), to_dev(v)
    wsb = ops.flash_decode_workspace_bytes(batch, g, Hkv, 128, fits)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda")
    want, got = dev_empty(q.shape), dev_empty(q.shape)
    ops.hip_flash_decode_gqa_layer(want, dq, dk, dv, ws, wsb, batch, n, n, g, Hkv, 128, fits, dt)
    ops.hip_flash_decode_gqa_static_layer(got, dq, dk, dv, batch, n, n, g, Hkv, 128, 0, dt)
    torch.cuda.synchronize()
    assert np.array_equal(to_host(got), to_host(want))

