"""twg_masked_select_f32_static: the entry point that allocates nothing (its tickets and
status words live in a device array inside the library) must give exactly what
twg_masked_select_f32 gives with a caller-allocated scratch buffer: same count, same
values in the same order, bit for bit.  Two calls in a row share the array, the second
on a smaller input, so what the first call left behind must not leak into the second."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(twg, L, n, p, seed):
    g = torch.Generator().manual_seed(seed)
    src = torch.rand(n, generator=g) * 2 - 1
    mask = torch.rand(n, generator=g) < p
    d_src, d_mask = twg.to_device(src), twg.to_device(mask)
    it = twg.dense_iter(n)
    res = []
    for static in (False, True):
        out = twg.DeviceBuffer(4 * n + 256)
        cnt = twg.DeviceBuffer(8)
        twg.check(L.twg_fill_bytes(out.ptr, 0xAB, out.nbytes, None))
        if static:
            before = twg.mem_stats()
            twg.check(L.twg_masked_select_f32_static(out.ptr, cnt.ptr, d_src.ptr, d_mask.ptr,
                                                     ctypes.byref(it), None))
            after = twg.mem_stats()
            assert after == before, "the call went to the allocator"
        else:
            sb = L.twg_masked_select_scratch_bytes(n)
            scratch = twg.DeviceBuffer(sb)
            twg.check(L.twg_masked_select_f32(out.ptr, cnt.ptr, d_src.ptr, d_mask.ptr,
                                              ctypes.byref(it), scratch.ptr, sb, None))
        k = int(cnt.download((1,), torch.int64)[0])
        raw = out.download((out.nbytes,), torch.uint8)
        res.append((k, raw))
    (k0, raw0), (k1, raw1) = res
    assert k0 == int(mask.sum()) == k1
    # the k values and the untouched bytes behind them
    assert torch.equal(raw0, raw1)
    assert torch.equal(raw1[:4 * k1].view(torch.float32), src[mask])
    return k1


def test_static_scratch_matches_allocated_scratch(twg):
    L = twg.load()
    print("static masked_select: 2^22+12345 elements, then 70001", flush=True)
    # streaming kernel with an incomplete last tile (the ticket and thousands of status words
    # are left behind) ...
    _both(twg, L, (1 << 22) + 12345, 0.5, 1)
    # ... then a smaller input that reuses the front of the same array
    _both(twg, L, 70001, 0.3, 2)
    # and a third that fits one tile (no ticket, no look-back)
    _both(twg, L, 1000, 0.9, 3)


def test_static_scratch_limits(twg):
    L = twg.load()
    it = twg.dense_iter(twg.MS_STATIC_MAX_NUMEL + 1)
    buf = twg.DeviceBuffer(64)
    rc = L.twg_masked_select_f32_static(buf.ptr, buf.ptr, buf.ptr, buf.ptr, ctypes.byref(it), None)
    assert rc == twg.E_TOO_LARGE
    assert b"limit" in L.twg_error_string(rc)
    # an empty input writes a count of zero and touches nothing else
    it0 = twg.dense_iter(0)
    cnt = twg.DeviceBuffer(8)
    twg.check(L.twg_fill_bytes(cnt.ptr, 0xFF, 8, None))
    twg.check(L.twg_masked_select_f32_static(None, cnt.ptr, None, None, ctypes.byref(it0), None))
    assert int(cnt.download((1,), torch.int64)[0]) == 0
