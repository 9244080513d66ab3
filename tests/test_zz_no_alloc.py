"""twg_masked_select_f32_static: the entry point that allocates nothing (its tickets and
status words live in a device array inside the library) must give exactly what
twg_masked_select_f32 gives with a caller-allocated scratch buffer: same count, same
values in the same order, bit for bit.  Two calls in a row share the array, the second
on a smaller input, so what the first call left behind must not leak into the second."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

_hip = None


def _free_device_bytes():
    """Free device memory as the driver reports it (hipMemGetInfo): unlike the allocator's
    own counters it also sees a hipMalloc made behind the allocator's back."""
    global _hip
    if _hip is None:
        _hip = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert _hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def _both(twg, L, n, p, seed, shift=0):
    """shift: elements the source pointer is moved off its 16-byte alignment (the
    one-element-per-lane variant of the kernel then runs, on the same static array)."""
    g = torch.Generator().manual_seed(seed)
    src_all = torch.rand(n + shift, generator=g) * 2 - 1
    src = src_all[shift:]
    mask = torch.rand(n, generator=g) < p
    d_src_buf, d_mask = twg.to_device(src_all), twg.to_device(mask)
    d_src = d_src_buf.at(4 * shift)
    it = twg.dense_iter(n)
    res = []
    for static in (False, True):
        out = twg.DeviceBuffer(4 * n + 256)
        cnt = twg.DeviceBuffer(8)
        twg.check(L.twg_fill_bytes(out.ptr, 0xAB, out.nbytes, None))
        if static:
            twg.sync()
            before, free_before = twg.mem_stats(), _free_device_bytes()
            twg.check(L.twg_masked_select_f32_static(out.ptr, cnt.ptr, d_src, d_mask.ptr,
                                                     ctypes.byref(it), None))
            after, free_after = twg.mem_stats(), _free_device_bytes()
            assert after == before, "the call went to the allocator"
            assert free_after == free_before, "the call allocated or freed device memory"
        else:
            sb = L.twg_masked_select_scratch_bytes(n)
            scratch = twg.DeviceBuffer(sb)
            twg.check(L.twg_masked_select_f32(out.ptr, cnt.ptr, d_src, d_mask.ptr,
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
    # a source that is not 16-byte aligned: the one-element-per-lane variant, several tiles
    _both(twg, L, 5 * 16384 + 77, 0.4, 4, shift=1)
    _both(twg, L, 40000, 0.6, 5, shift=3)


def test_static_scratch_is_not_cleared_between_calls(twg):
    # Calls in a row on the library's array, which no launch clears in between: each launch
    # tells its status words from its predecessors' by their epoch and counts its tiles from
    # where the ticket counter stands.  Sizes that take the streaming kernel (thousands of
    # status words), the small-tile kernel, a single tile (no ticket drawn) and the
    # one-element-per-lane kernel, growing and shrinking, every density; also through the entry
    # point that hands the count to the host, for other element sizes and with layouts that are
    # copied dense first.
    L = twg.load()
    g = torch.Generator().manual_seed(2024)
    sizes = [(1 << 21) + 5, 70001, (1 << 23) + 999, 8192, 300000, (1 << 22), 1000, 65536 * 3 + 1,
             (1 << 21) + 5, 100, 40000, (1 << 24) + 17, 20000]
    for i, n in enumerate(sizes):
        p = (0.02, 0.5, 0.97, 0.3)[i % 4]
        shift = 1 if i % 5 == 4 else 0
        print(f"static call {i}: n={n} p={p} shift={shift}", flush=True)
        src_all = torch.rand(n + shift, generator=g)
        src, mask = src_all[shift:], torch.rand(n, generator=g) < p
        d_src, d_mask = twg.to_device(src_all), twg.to_device(mask)
        out, cnt = twg.DeviceBuffer(4 * n + 256), twg.DeviceBuffer(8)
        it = twg.dense_iter(n)
        if i % 3 == 2:
            kh = ctypes.c_int64(-7)
            twg.check(L.twg_masked_select_count(out.ptr, ctypes.byref(kh), d_src.at(4 * shift), 4, d_mask.ptr,
                                                ctypes.byref(it), None, 0, None))
            k = kh.value
        else:
            twg.check(L.twg_masked_select_f32_static(out.ptr, cnt.ptr, d_src.at(4 * shift), d_mask.ptr,
                                                     ctypes.byref(it), None))
            k = int(cnt.download((1,), torch.int64)[0])
        assert k == int(mask.sum()), (i, n, k)
        assert torch.equal(out.download((k,), torch.float32), src[mask]), (i, n)
    # other element sizes and a transposed source through the count entry point
    import capi_helpers as H
    for dtype in (torch.int64, torch.uint8, torch.int16, torch.float32):
        x = (torch.randn(700, 500, generator=g) * 100).to(dtype).t()
        m = torch.rand(500, 700, generator=g) < 0.4
        vals, k = H.masked_select_on_library_array(x, m)
        assert k == int(m.sum()) and torch.equal(vals, torch.masked_select(x, m)), dtype


def test_library_array_from_two_host_threads(twg):
    # Two host threads call into the array at once (ctypes drops the GIL for the call): the
    # epoch and ticket bookkeeping is taken under the array's lock together with the launch, so
    # every call still sees its own count and values.
    import threading
    L = twg.load()
    errors = []

    def worker(seed):
        try:
            g = torch.Generator().manual_seed(seed)
            for i in range(12):
                n = (70001, (1 << 21) + 3, 9000, 300000)[i % 4] + seed
                src, mask = torch.rand(n, generator=g), torch.rand(n, generator=g) < (0.2 + 0.05 * i)
                d_src, d_mask = twg.to_device(src), twg.to_device(mask)
                out = twg.DeviceBuffer(4 * n + 256)
                it = twg.dense_iter(n)
                kh = ctypes.c_int64(-7)
                twg.check(L.twg_masked_select_count(out.ptr, ctypes.byref(kh), d_src.ptr, 4, d_mask.ptr,
                                                    ctypes.byref(it), None, 0, None))
                if kh.value != int(mask.sum()) or not torch.equal(out.download((kh.value,), torch.float32), src[mask]):
                    errors.append((seed, i, n, kh.value))
        except Exception as e:  # noqa: BLE001 - reported below, in the test's thread
            errors.append((seed, repr(e)))

    threads = [threading.Thread(target=worker, args=(s,)) for s in (1, 2)]
    print("library array: two host threads", flush=True)
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_static_scratch_is_refused_to_a_second_stream_while_in_use(twg):
    # One array per GPU: a call on another stream while the previous call's kernels may still
    # be running must be refused (TWG_E_BUSY), not left to corrupt the tickets; once that work
    # has finished the other stream is served.
    L = twg.load()
    hip = ctypes.CDLL("libamdhip64.so")
    stream_a, stream_b = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipStreamCreateWithFlags(ctypes.byref(stream_a), 1) == 0  # hipStreamNonBlocking
    assert hip.hipStreamCreateWithFlags(ctypes.byref(stream_b), 1) == 0
    n = (1 << 22) + 777
    g = torch.Generator().manual_seed(8)
    src, mask = torch.rand(n, generator=g), torch.rand(n, generator=g) < 0.5
    d_src, d_mask = twg.to_device(src), twg.to_device(mask)
    out_a, out_b = twg.DeviceBuffer(4 * n), twg.DeviceBuffer(4 * n)
    cnt_a, cnt_b = twg.DeviceBuffer(8), twg.DeviceBuffer(8)
    big = twg.DeviceBuffer(1 << 30)
    it = twg.dense_iter(n)
    twg.sync()
    # ~20 ms of fills keep stream A busy, the static call queues up behind them
    print("static masked_select: second stream while the first is busy", flush=True)
    for _ in range(60):
        twg.check(L.twg_fill_bytes(big.ptr, 1, big.nbytes, stream_a))
    twg.check(L.twg_masked_select_f32_static(out_a.ptr, cnt_a.ptr, d_src.ptr, d_mask.ptr,
                                             ctypes.byref(it), stream_a))
    rc = L.twg_masked_select_f32_static(out_b.ptr, cnt_b.ptr, d_src.ptr, d_mask.ptr,
                                        ctypes.byref(it), stream_b)
    assert rc == twg.E_BUSY, rc
    assert b"another stream" in L.twg_error_string(rc)
    # the same stream is never refused: its calls are ordered
    twg.check(L.twg_masked_select_f32_static(out_a.ptr, cnt_a.ptr, d_src.ptr, d_mask.ptr,
                                             ctypes.byref(it), stream_a))
    assert hip.hipStreamSynchronize(stream_a) == 0
    twg.check(L.twg_masked_select_f32_static(out_b.ptr, cnt_b.ptr, d_src.ptr, d_mask.ptr,
                                             ctypes.byref(it), stream_b))
    assert hip.hipStreamSynchronize(stream_b) == 0
    k = int(mask.sum())
    for cnt, out in ((cnt_a, out_a), (cnt_b, out_b)):
        assert int(cnt.download((1,), torch.int64)[0]) == k
        assert torch.equal(out.download((k,), torch.float32), src[mask])
    assert hip.hipStreamDestroy(stream_a) == 0 and hip.hipStreamDestroy(stream_b) == 0


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


def test_static_scratch_under_graph_capture_then_eager(twg):
    # A graph that holds a launch on the library's array replays it with the arguments of its
    # capture, so from the first call under capture on every call clears what it needs again.
    # Eager calls, a captured call replayed with new contents, eager calls again: all exact.
    hip = ctypes.CDLL("libamdhip64.so")
    L = twg.load()
    g = torch.Generator().manual_seed(555)

    def eager(n, p):
        src, mask = torch.rand(n, generator=g), torch.rand(n, generator=g) < p
        d_src, d_mask = twg.to_device(src), twg.to_device(mask)
        out, cnt = twg.DeviceBuffer(4 * n + 256), twg.DeviceBuffer(8)
        it = twg.dense_iter(n)
        twg.check(L.twg_masked_select_f32_static(out.ptr, cnt.ptr, d_src.ptr, d_mask.ptr, ctypes.byref(it), None))
        k = int(cnt.download((1,), torch.int64)[0])
        assert k == int(mask.sum()) and torch.equal(out.download((k,), torch.float32), src[mask]), (n, p)

    eager((1 << 21) + 77, 0.5)
    eager(90000, 0.2)
    stream = ctypes.c_void_p()
    assert hip.hipStreamCreateWithFlags(ctypes.byref(stream), 1) == 0  # hipStreamNonBlocking
    n = (1 << 21) + 4096 + 13
    src, mask = torch.rand(n, generator=g), torch.rand(n, generator=g) < 0.37
    d_src, d_mask = twg.to_device(src), twg.to_device(mask)
    out, cnt = twg.DeviceBuffer(4 * n + 256), twg.DeviceBuffer(8)
    it = twg.dense_iter(n)
    twg.sync()
    assert hip.hipStreamBeginCapture(stream, 1) == 0  # hipStreamCaptureModeThreadLocal
    try:
        rc = L.twg_masked_select_f32_static(out.ptr, cnt.ptr, d_src.ptr, d_mask.ptr, ctypes.byref(it), stream)
    finally:
        graph = ctypes.c_void_p()
        rc_end = hip.hipStreamEndCapture(stream, ctypes.byref(graph))
    assert rc == 0 and rc_end == 0, (rc, rc_end)
    graph_exec = ctypes.c_void_p()
    assert hip.hipGraphInstantiate(ctypes.byref(graph_exec), graph, None, None, ctypes.c_size_t(0)) == 0
    try:
        for rep in range(3):
            print(f"static masked_select: graph replay {rep}", flush=True)
            if rep:
                src, mask = torch.rand(n, generator=g), torch.rand(n, generator=g) < (0.1 + 0.4 * rep)
                d_src.upload(src)
                d_mask.upload(mask)
                eager(50000 * rep + 3, 0.6)   # eager work on the array between the replays
            twg.sync()
            assert hip.hipGraphLaunch(graph_exec, stream) == 0
            assert hip.hipStreamSynchronize(stream) == 0
            k = int(cnt.download((1,), torch.int64)[0])
            assert k == int(mask.sum()), (rep, k)
            assert torch.equal(out.download((k,), torch.float32), src[mask]), rep
    finally:
        hip.hipGraphExecDestroy(graph_exec)
        hip.hipGraphDestroy(graph)
        hip.hipStreamDestroy(stream)
    eager((1 << 22) + 5, 0.9)
    eager(70001, 0.4)
