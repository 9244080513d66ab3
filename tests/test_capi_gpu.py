"""Parity of the HIP kernels, driven through the C ABI of libtwg_hip.so, against the
CPU oracle (and ATen's CPU kernels where those are the reference's implementation).

Bars: bit-exact for add (alpha = 1 and alpha != 1, same two roundings as the
oracle), relu, copy, eq, ne, bitwise_and and masked_select (length and order);
|got - ref| <= 2e-6*|ref| + 4 subnormal steps for gelu and silu against the
closed form.
"""
import ctypes
import os
import itertools

import pytest
import torch
import torch.nn.functional as F

import capi_helpers as H
import twg_workloads as W
from oracle import oracle
from util import (FLOOR, bit_equal, closed_form64, load_activation_golden, rel_err_ok, ulp_diff)

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)


# ----------------------------------------------------------------- runtime

def test_device_is_mi355x(twg):
    name, cus, mem = twg.device_info()
    _say(f"device: {name}, {cus} CUs, {mem / 2**30:.0f} GiB")
    assert "gfx950" in name
    assert cus >= 200


def test_allocator_caches_and_handles_zero(twg):
    L = twg.load()
    p = ctypes.c_void_p(1)
    twg.check(L.twg_malloc(ctypes.byref(p), 0))
    assert not p.value  # zero bytes -> NULL, success
    before = twg.mem_stats()
    a = twg.DeviceBuffer(3 << 20)
    addr = a.ptr
    a.free()
    b = twg.DeviceBuffer(3 << 20)
    after = twg.mem_stats()
    assert b.ptr == addr, "a freed block of the same size class is handed out again"
    assert after["n_cache_hits"] >= before["n_cache_hits"] + 1
    assert L.twg_free(ctypes.c_void_p(12345)) == twg.E_INVALID_ARG  # not ours
    b.free()


def test_copy_round_trip_fp32_and_bool(twg):
    g = torch.Generator().manual_seed(1)
    # 80 MiB wraps the ring of pinned staging slots several times, with a ragged tail
    for t in (torch.randn((80 << 20) // 4 + 3, generator=g),
              torch.rand(1000003, generator=g) < 0.5,
              torch.randn(5, generator=g)):
        buf = twg.to_device(t)
        back = buf.download(t.shape, t.dtype)
        assert bit_equal(back, t)
    # large copies into and out of host ranges that start at odd addresses
    raw = torch.randint(0, 256, ((40 << 20) + 77,), dtype=torch.uint8, generator=g)
    L = twg.load()
    for off in (1, 15, 16, 33):
        nb = raw.numel() - off - 5
        dev = twg.DeviceBuffer(nb)
        twg.check(L.twg_memcpy_h2d(dev.ptr, raw.data_ptr() + off, nb, None))
        back = torch.full((raw.numel(),), 0xEE, dtype=torch.uint8)
        twg.check(L.twg_memcpy_d2h(back.data_ptr() + off, dev.ptr, nb, None))
        assert torch.equal(back[off:off + nb], raw[off:off + nb])
        assert bool((back[:off] == 0xEE).all()) and bool((back[off + nb:] == 0xEE).all())
        dev.free()
    # reads of up to 16 KiB take a different route back than larger ones
    small = twg.to_device(raw[:65536])
    for nb in (1, 3, 8, 255, 256, 257, 1025, 4096, 16383, 16384, 16385, 20000):
        for off in (0, 1, 4, 7):
            back = torch.full((nb + 16,), 0xEE, dtype=torch.uint8)
            twg.check(L.twg_memcpy_d2h(back.data_ptr() + 5, small.ptr + off, nb, None))
            assert torch.equal(back[5:5 + nb], raw[off:off + nb])
            assert bool((back[:5] == 0xEE).all()) and bool((back[5 + nb:] == 0xEE).all())
    # uploads of a few bytes travel as a kernel argument: every size around the switch, at odd
    # device and host offsets, must leave the neighbouring bytes alone
    for nb in (1, 2, 3, 4, 8, 63, 64, 65, 255, 256, 257, 300, 1023, 1024, 1025, 1500):
        for off in (0, 1, 5):
            twg.check(L.twg_fill_bytes(small.ptr, 0xEE, 4096, None))
            twg.check(L.twg_memcpy_h2d(small.ptr + 16 + off, raw.data_ptr() + 3 + off, nb, None))
            back = small.download((2048,), torch.uint8)
            assert torch.equal(back[16 + off:16 + off + nb], raw[3 + off:3 + off + nb]), (nb, off)
            assert bool((back[:16 + off] == 0xEE).all()) and bool((back[16 + off + nb:] == 0xEE).all())
    # device -> device and fill
    t = torch.randn(4097, generator=g)
    src = twg.to_device(t)
    dst = twg.DeviceBuffer(t.numel() * 4 + 16)
    L = twg.load()
    twg.check(L.twg_fill_bytes(dst.ptr, 0xAB, dst.nbytes, None))
    twg.check(L.twg_memcpy_d2d(dst.ptr + 8, src.ptr, t.numel() * 4, None))
    raw = dst.download((dst.nbytes,), torch.uint8)
    assert bool((raw[:8] == 0xAB).all()) and bool((raw[-8:] == 0xAB).all())
    assert bit_equal(raw[8:-8].view(torch.float32), t)


def test_large_device_to_device_copies(twg):
    # from 128 MiB on, aligned copies run the library's own streaming copy kernel and hand a
    # tail of 1-3 bytes to the runtime; misaligned ones stay with the runtime
    L = twg.load()
    nb = (1 << 27) + 4096 + 3
    g = torch.Generator().manual_seed(5)
    host = torch.randint(0, 256, (nb + 64,), dtype=torch.uint8, generator=g)
    src = twg.to_device(host)
    dst = twg.DeviceBuffer(nb + 128)
    for d_off, s_off in ((16, 0), (16, 16), (17, 0), (16, 1), (32, 48)):
        _say(f"d2d {nb} bytes, offsets {d_off}/{s_off}")
        twg.check(L.twg_fill_bytes(dst.ptr, 0xCD, dst.nbytes, None))
        twg.check(L.twg_memcpy_d2d(dst.ptr + d_off, src.ptr + s_off, nb, None))
        raw = dst.download((dst.nbytes,), torch.uint8)
        assert torch.equal(raw[d_off:d_off + nb], host[s_off:s_off + nb]), (d_off, s_off)
        assert bool((raw[:d_off] == 0xCD).all()) and bool((raw[d_off + nb:] == 0xCD).all())


def test_copy_sizes_around_every_staging_boundary(twg):
    # The pinned ring is divided differently for each copy size and large copies are split
    # over helper threads; sizes just below, at and above each switch, with ragged tails, in
    # an order that changes the division between consecutive copies and leaves uploads in
    # flight when the next copy starts.
    L = twg.load()
    g = torch.Generator().manual_seed(77)
    mib = 1 << 20
    sizes = [mib - 1, mib, mib + 1, 2 * mib + 3, 4 * mib, 8 * mib - 1, 8 * mib, 8 * mib + 5,
             16 * mib - 7, 16 * mib + mib + 3, 32 * mib - 1, 32 * mib + 12, 9 * mib + 999,
             128 * mib - 3, 128 * mib + 16 * mib + 11, 300, 64 * mib + 1]
    raw = torch.randint(0, 256, (max(sizes) + 64,), dtype=torch.uint8, generator=g)
    back = torch.empty(max(sizes) + 64, dtype=torch.uint8)
    dev = twg.DeviceBuffer(max(sizes))
    small = twg.DeviceBuffer(4096)
    for i, nb in enumerate(sizes):
        _say(f"copy {nb} bytes")
        off = (i * 7) % 31
        twg.check(L.twg_memcpy_h2d(dev.ptr, raw.data_ptr() + off, nb, None))
        if i % 2:  # a small upload of another division right behind the large one
            twg.check(L.twg_memcpy_h2d(small.ptr, raw.data_ptr(), 4096, None))
        back.fill_(0xEE)
        twg.check(L.twg_memcpy_d2h(back.data_ptr() + 3, dev.ptr, nb, None))
        assert torch.equal(back[3:3 + nb], raw[off:off + nb]), nb
        assert bool((back[:3] == 0xEE).all()) and bool((back[3 + nb:3 + nb + 61] == 0xEE).all()), nb


def test_uploads_through_the_outbox(twg):
    # Uploads of 1 KiB..2 MiB are copied into pinned slots (up to 16 at a time) and fetched by a
    # kernel, one workgroup per slot, that then releases them: every size class and destination alignment, many more uploads in a row
    # than there are slots (each to its own place, checked at the end), and uploads queued
    # behind a long kernel, so that the host has to wait for a slot.
    L = twg.load()
    g = torch.Generator().manual_seed(123)
    raw = torch.randint(0, 256, ((1 << 21) + 64,), dtype=torch.uint8, generator=g)
    dev = twg.DeviceBuffer((1 << 21) + 128)
    back = torch.empty((1 << 21) + 128, dtype=torch.uint8)
    for nb in (1025, 1040, 2048, 4096, 4099, 16384, 40000, 65535, 65536, 65537, 100000, 262143, 262144, 262145,
               300001, 524288, 786433, (1 << 20) - 1, 1 << 20, (1 << 20) + 16385, (1 << 21) - 3, 1 << 21, (1 << 21) + 1):
        for dst_off in (0, 4, 16, 3):
            twg.check(L.twg_fill_bytes(dev.ptr, 0xEE, nb + 64, None))
            twg.check(L.twg_memcpy_h2d(dev.ptr + dst_off, raw.data_ptr() + 5, nb, None))
            twg.check(L.twg_memcpy_d2h(back.data_ptr(), dev.ptr, nb + 64, None))
            assert torch.equal(back[dst_off:dst_off + nb], raw[5:5 + nb]), (nb, dst_off)
            assert bool((back[:dst_off] == 0xEE).all()) and bool((back[dst_off + nb:nb + 64] == 0xEE).all()), (nb, dst_off)
    # 100 uploads of 8 KiB back to back, the host buffer overwritten right after each call
    piece = 8192
    scratch = torch.empty(piece, dtype=torch.uint8)
    for i in range(100):
        scratch.copy_(raw[i * piece:(i + 1) * piece])
        twg.check(L.twg_memcpy_h2d(dev.ptr + i * piece, scratch.data_ptr(), piece, None))
        scratch.fill_(0)
    twg.check(L.twg_memcpy_d2h(back.data_ptr(), dev.ptr, 100 * piece, None))
    assert torch.equal(back[:100 * piece], raw[:100 * piece])
    # small and large uploads interleaved, so that groups of four start at either half
    sizes = [3000, 200000, 70000, 5000, 5000, 262144, 1500, 400000, 65536, 131073]
    offs, pos = [], 0
    for nb in sizes:
        offs.append(pos)
        pos += (nb + 63) // 64 * 64
    for rep in range(3):
        for nb, o in zip(sizes, offs):
            twg.check(L.twg_memcpy_h2d(dev.ptr + o, raw.data_ptr() + o + rep, nb, None))
        twg.check(L.twg_memcpy_d2h(back.data_ptr(), dev.ptr, pos, None))
        for nb, o in zip(sizes, offs):
            assert torch.equal(back[o:o + nb], raw[o + rep:o + rep + nb]), (rep, nb)
    # the same behind a kernel that keeps the stream busy for a while
    n = 1 << 27
    big_a, big_o = twg.DeviceBuffer(4 * n), twg.DeviceBuffer(4 * n)
    it = twg.make_iter([n], [1], [1])
    for _ in range(4):
        twg.check(L.twg_unary_f32(twg.UNARY_GELU_ERF, big_o.ptr, big_a.ptr, ctypes.byref(it), None))
    for i in range(40):
        scratch.copy_(raw[(i + 7) * piece:(i + 8) * piece])
        twg.check(L.twg_memcpy_h2d(dev.ptr + i * piece, scratch.data_ptr(), piece, None))
        scratch.fill_(1)
    twg.check(L.twg_memcpy_d2h(back.data_ptr(), dev.ptr, 40 * piece, None))
    assert torch.equal(back[:40 * piece], raw[7 * piece:47 * piece])


def test_copies_with_a_small_pinned_ring(twg):
    # TWG_STAGE_RING_MIB shrinks the pinned ring (what the library also does by itself when
    # 64 MiB cannot be pinned): every copy size must still round-trip.  The variable is read
    # when the ring is created, hence a process of its own.
    import subprocess
    import sys
    code = r"""
import sys, ctypes, torch
sys.path.insert(0, sys.argv[1])
import twg_capi as capi
L = capi.load(); capi.init()
g = torch.Generator().manual_seed(5)
mib = 1 << 20
raw = torch.randint(0, 256, (40 * mib + 200,), dtype=torch.uint8, generator=g)
back = torch.empty_like(raw)
dev = capi.DeviceBuffer(raw.numel())
for nb in (300, 70000, mib + 1, 3 * mib + 7, 4 * mib, 4 * mib + 1, 9 * mib + 5, 40 * mib + 99):
    capi.check(L.twg_memcpy_h2d(dev.ptr, raw.data_ptr() + 1, nb - 1, None))
    back.fill_(0xEE)
    capi.check(L.twg_memcpy_d2h(back.data_ptr() + 2, dev.ptr, nb - 1, None))
    assert torch.equal(back[2:nb + 1], raw[1:nb]), nb
    assert int(back[1]) == 0xEE and int(back[nb + 1]) == 0xEE, nb
print("small ring ok")
"""
    env = dict(os.environ, TWG_STAGE_RING_MIB="4")
    pkg = os.path.dirname(os.path.abspath(twg.__file__))
    r = subprocess.run([sys.executable, "-c", code, pkg], env=env, capture_output=True, text=True,
                       timeout=150)
    assert r.returncode == 0 and "small ring ok" in r.stdout, r.stdout + r.stderr


# --------------------------------------------------------------------- add

def test_add_config1_contiguous(twg):
    a, b = W.add_contiguous(1 << 20, seed=0)
    got = H.add(a, b)
    assert bit_equal(got, oracle.add(a, b))
    assert bit_equal(got, a + b)


@pytest.mark.parametrize("n", [0, 1, 3, 4, 5, 1023, 1024, 4095, 4096, 4097, 8191, 65536 + 13,
                               (1 << 20) + 7])
def test_add_ragged_sizes_and_misaligned(twg, n):
    g = torch.Generator().manual_seed(n)
    a = torch.randn(n + 3, generator=g)
    b = torch.randn(n + 3, generator=g)
    assert bit_equal(H.add(a[:n], b[:n]), a[:n] + b[:n])
    # storage offsets 1 and 3: pointers no longer 16-byte aligned
    out = torch.zeros(n + 2)[2:]
    got = H.add(a[1:n + 1], b[3:n + 3], out=out)
    assert bit_equal(got, a[1:n + 1] + b[3:n + 3])


@pytest.mark.parametrize("alpha", [1.0, -1.0, 0.5, 1.7, 3.14159, 0.0])
def test_add_alpha_matches_oracle_bits(twg, alpha):
    g = torch.Generator().manual_seed(7)
    a = torch.randn(100003, generator=g)
    b = torch.randn(100003, generator=g)
    got = H.add(a, b, alpha=alpha)
    assert bit_equal(got, oracle.add(a, b, alpha=alpha))
    # and within 1 ulp of the exactly rounded value where nothing cancels
    pa, pb = a.abs() + 0.5, b.abs() + 0.5
    af = float(torch.tensor(abs(alpha), dtype=torch.float32))
    ref = (pa.double() + af * pb.double()).float()
    assert ulp_diff(H.add(pa, pb, alpha=abs(alpha)), ref) <= 1


def test_add_special_values(twg):
    s = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), float("nan"), 1e-45, -1e-45, 3e38,
                      1.17e-38])
    a = s.repeat_interleave(s.numel())
    b = s.repeat(s.numel())
    assert ulp_diff(H.add(a, b), a + b) == 0
    got, ref = H.add(a, b), a + b
    ok = ~torch.isnan(ref)
    assert torch.equal(torch.signbit(got[ok]), torch.signbit(ref[ok]))


@pytest.mark.parametrize("rows,cols", [(256, 4096), (37, 1000), (5, 64), (3, 70001), (1, 513)])
def test_add_row_and_column_bias(twg, rows, cols):
    # config 3a shape family: [rows, cols] + [1, cols]; plus the column-bias and
    # scalar-broadcast variants
    a, bias, _ = W.broadcast_add_inputs(rows, cols, seed=rows)
    assert bit_equal(H.add(a, bias), oracle.add(a, bias))
    assert bit_equal(H.add(bias, a), bias + a)
    col = bias[0, :rows].reshape(rows, 1).contiguous() if rows <= cols else a[:, :1].contiguous()
    assert bit_equal(H.add(a, col), a + col)
    assert bit_equal(H.add(a, a[0, 0].reshape(1, 1)), a + a[0, 0])
    # outer-strided rows (every other row of a taller matrix)
    tall = torch.cat([a, a * 2.0], 0)
    assert bit_equal(H.add(tall[::2], bias), tall[::2] + bias)


@pytest.mark.parametrize("rows,cols", [(256, 512), (100, 70), (64, 64), (65, 33), (16, 1000),
                                       # multiples of 4 take the 128-bit tile kernel: full and
                                       # ragged 256x32 tiles, and the 64x64 shape below 256
                                       (264, 300), (68, 132), (36, 1028), (1024, 40), (20, 16)])
def test_add_transposed_operand(twg, rows, cols):
    # config 3b shape family: A[rows, cols] viewed as (cols, rows) with strides
    # (1, cols), plus a contiguous C[cols, rows].  TensorIterator gives the output
    # the layout of the first input, so both output layouts are covered.
    a, _, c = W.broadcast_add_inputs(rows, cols, seed=cols)
    at = a.as_strided((cols, rows), (1, cols))
    ref = oracle.add(at, c)
    assert bit_equal(ref, at + c)
    out_like_a = torch.zeros(rows, cols).t()  # strides (1, cols)
    got = H.add(at, c, out=out_like_a)
    assert bit_equal(got.contiguous(), ref)
    got2 = H.add(at, c)  # contiguous output: now `at` is the transposed one
    assert bit_equal(got2, ref)
    got3 = H.add(c, at)
    assert bit_equal(got3, ref)
    # batched: leading dimension on top of the transposed pair
    a3 = torch.stack([a, a + 1.0, a - 1.0])
    at3 = a3.transpose(1, 2)
    c3 = torch.stack([c, c * 2.0, c * 0.5])
    assert bit_equal(H.add(at3, c3), at3 + c3)


@pytest.mark.parametrize("shape,order", [
    # an operand stored with a short innermost extent that is another dimension than the
    # output's innermost one, the next memory dimension yet another: (3 channels, a head
    # size of 16, 56) x (20..40) walked as one transposed dimension
    ((6, 3, 20, 96), (3, 0, 2, 1)), ((6, 3, 20, 96), (0, 3, 2, 1)), ((5, 16, 24, 64), (3, 0, 2, 1)),
    ((3, 56, 9, 96), (0, 3, 2, 1)), ((4, 3, 37, 260), (3, 0, 2, 1)), ((2, 7, 33, 300), (0, 3, 2, 1)),
    ((2, 3, 5, 20), (3, 0, 2, 1)),
    # batched transposes whose extents and row pitches are not multiples of 4
    ((4, 197, 72), (0, 2, 1)), ((3, 66, 259), (0, 2, 1)), ((2, 261, 35), (0, 2, 1)),
    ((5, 19, 1030), (0, 2, 1)), ((300, 77), (1, 0)), ((67, 513), (1, 0)),
    # dimension 0 of 96..192 elements: the 128 x 64 tile shape
    ((3, 40, 7, 96), (3, 2, 1, 0)), ((2, 70, 160), (2, 1, 0)), ((130, 192), (1, 0)),
    # stored [.., x, c] with a short c, wanted [.., c, x]: strips through LDS
    ((5, 3, 40, 96), (0, 2, 3, 1)), ((5, 3, 40, 96), (2, 0, 3, 1)), ((3, 1000), (1, 0)),
    ((4, 4, 1027), (0, 2, 1)), ((2, 16, 700), (0, 2, 1)), ((2, 32, 301), (0, 2, 1)),
    ((2, 33, 300), (0, 2, 1)), ((7, 2, 5000), (0, 2, 1)), ((3, 5, 255), (0, 2, 1)),
    ((2, 8, 3001), (0, 2, 1)), ((3, 16, 1100), (0, 2, 1)), ((2, 24, 777), (0, 2, 1)),
    # the mirror image: the output [.., x, c] with a short c, the operand stored planar [.., c, x]
    # (NCHW -> NHWC with few channels): strips interleaved through LDS
    ((4, 30, 40, 3), (0, 3, 1, 2)), ((2, 1000, 3), (0, 2, 1)), ((1027, 4), (1, 0)), ((3, 700, 16), (0, 2, 1)),
    ((2, 301, 31), (0, 2, 1)), ((5000, 2), (1, 0)), ((3, 2051, 7), (0, 2, 1)), ((2, 4099, 24), (0, 2, 1)),
    ((2, 3, 255, 5), (0, 1, 3, 2)), ((2, 2, 260, 8), (1, 0, 3, 2)), ((300, 32), (1, 0)),
    # 32 to 63 channels take the same strips (32 values of x each)
    ((2, 301, 33), (0, 2, 1)), ((3, 700, 48), (0, 2, 1)), ((2, 40, 50, 63), (0, 3, 1, 2)), ((1027, 36), (1, 0)),
    # a short x: several strips per block (groups of the next dimension, the last group shorter)
    ((7, 5, 40, 3), (0, 1, 3, 2)), ((3, 11, 100, 2), (0, 1, 3, 2)), ((2, 9, 33, 31), (0, 1, 3, 2)),
    ((2, 23, 56, 3), (1, 0, 3, 2)), ((40, 112, 3), (0, 2, 1)), ((1, 3, 32, 4), (0, 1, 3, 2)),
    # channels-last pixels with two outer dimensions swapped: tiles of pixels through LDS (full
    # and ragged tiles, channel counts that do and do not divide a pack, the transposed
    # dimension next to x or further out)
    ((4, 30, 40, 3), (0, 2, 1, 3)), ((5, 33, 35, 4), (0, 2, 1, 3)), ((37, 9, 45, 2), (2, 1, 0, 3)),
    ((3, 70, 65, 7), (0, 2, 1, 3)), ((2, 19, 23, 16), (0, 2, 1, 3)), ((2, 40, 17, 31), (0, 2, 1, 3)),
    ((12, 13, 14, 5), (1, 2, 0, 3)), ((9, 8, 8, 24), (2, 0, 1, 3)), ((64, 65, 3), (1, 0, 2)),
    ((2, 3, 32, 64, 8), (0, 1, 3, 2, 4)), ((2, 100, 8, 3), (0, 2, 1, 3)),
    # the same with fewer than 256 elements per strip: several strips per block
    ((4, 3, 23, 100), (2, 0, 3, 1)), ((3, 5, 9, 33), (0, 2, 3, 1)), ((2, 2, 7, 250), (2, 0, 3, 1)),
    ((6, 3, 224), (0, 2, 1)), ((2, 31, 40), (0, 2, 1)), ((16, 3, 224, 96), (2, 0, 3, 1)),
    ((40, 3, 510), (0, 2, 1)),
    # short output rows (fewer than 256 elements) with the operand's unit stride along a
    # dimension beyond the second: the two innermost output dimensions walked as one, aligned
    # and ragged, one or two batch dimensions, merged extents that end inside a tile
    ((8, 130, 64, 64), (3, 2, 0, 1)), ((3, 40, 9, 64), (3, 2, 0, 1)), ((5, 33, 7, 50), (3, 2, 0, 1)),
    ((4, 64, 10, 96), (2, 3, 0, 1)), ((2, 3, 70, 5, 24), (0, 4, 3, 1, 2)), ((37, 11, 20), (2, 1, 0)),
    ((2, 100, 3, 85), (3, 2, 0, 1)),
    # a transposed extent of 33..64 elements under a wide dimension 0: one 64-wide tile along it
    ((64, 5, 8, 64), (1, 2, 3, 0)), ((64, 300), (1, 0)), ((48, 3, 520), (2, 1, 0)),
])
def test_add_permuted_operand_tiles(twg, shape, order):
    # `a` is stored with its dimensions in `order` (outermost first) and viewed in the logical
    # order; b and the output are contiguous.  Also with a in the second slot, with both inputs
    # permuted alike, and from storage offsets that break 16-byte alignment.
    g = torch.Generator().manual_seed(sum(shape) + order[0])
    phys = [shape[d] for d in order]
    inv = [order.index(d) for d in range(len(shape))]
    for off in (0, 1, 3):
        base = torch.randn(off + torch.Size(phys).numel(), generator=g)[off:].view(*phys)
        a = base.permute(*inv)
        assert tuple(a.shape) == tuple(shape)
        b = torch.randn(off + torch.Size(shape).numel(), generator=g)[off:].view(*shape)
        ref = oracle.add(a, b, alpha=0.75)
        assert bit_equal(H.add(a, b, alpha=0.75), ref)
        assert bit_equal(H.add(b, a, alpha=0.75), oracle.add(b, a, alpha=0.75))
        a2 = (base * 0.5 + 1.0).permute(*inv)
        assert bit_equal(H.add(a, a2, alpha=-1.25), oracle.add(a, a2, alpha=-1.25))
        out = torch.zeros(off + torch.Size(shape).numel())[off:].view(*shape)
        assert bit_equal(H.add(a, b, out=out), oracle.add(a, b))
        r = H.unary("twg_unary_f32", a, pre=(ctypes.c_int(1),))          # relu, contiguous output
        assert bit_equal(r, torch.relu(a))
        if off != 3:
            # a compare over the same layouts (its bools leave the tiles four to a dword); values
            # rounded to halves so that both outcomes occur
            ar, br = (a * 2).round(), (b * 2).round()
            assert ar.stride() == a.stride()
            assert torch.equal(H.binary("twg_eq_f32", ar, br, out_dtype=torch.bool), torch.eq(ar, br))
            assert torch.equal(H.binary("twg_eq_f32", br, ar, out_dtype=torch.bool), torch.eq(br, ar))


def test_fill_bytes_every_size_class(twg):
    # twg_fill_bytes: an unaligned head, a body of 16-byte packs and a tail.  From 16 MiB on the
    # body goes out in whole blocks of 4 KiB without a test per store, and what the last
    # whole block leaves over goes to the kernel for small fills: sizes on both sides of the
    # switch, at odd offsets, must set exactly their bytes.
    L = twg.load()
    mib = 1 << 20
    buf = twg.DeviceBuffer(49 * mib + 64)
    for nb in (0, 1, 15, 16, 17, 4097, 16 * mib - 1, 16 * mib, 16 * mib + 1, 16 * mib + 15,
               16 * mib + 4096 + 5, 16 * mib + 4080, 48 * mib + 1234567):
        for off in (0, 1, 7, 16):
            _say(f"fill {nb} bytes at offset {off}")
            twg.check(L.twg_fill_bytes(buf.ptr, 0xEE, buf.nbytes, None))
            twg.check(L.twg_fill_bytes(buf.ptr + off, 0x5A, nb, None))
            raw = buf.download((buf.nbytes,), torch.uint8)
            assert bool((raw[:off] == 0xEE).all()), (nb, off)
            assert bool((raw[off:off + nb] == 0x5A).all()), (nb, off)
            assert bool((raw[off + nb:] == 0xEE).all()), (nb, off)


@pytest.mark.parametrize("rows,cols", [(8, 64), (37, 128), (5, 4096), (16, 36), (3, 260), (64, 32), (2, 12288)])
def test_rows_stepped_by_two_and_three(twg, rows, cols):
    # x[:, ::2]: a lane fetches the two aligned packs that hold its four elements and keeps
    # every second value (x[:, ::3] stays with the gather and is checked beside it).  One or both inputs stepped, different steps, either
    # slot, rows that merge into one run, three dimensions, an activation over the view, views
    # that end with the storage's last element, and starts that break the 16-byte alignment
    # (those take the gather).
    g = torch.Generator().manual_seed(rows * 7 + cols)
    x2 = torch.randn(rows, 2 * cols, generator=g)
    x3 = torch.randn(rows, 3 * cols, generator=g)
    d = torch.randn(rows, cols, generator=g)
    a2, a3 = x2[:, ::2], x3[:, ::3]
    _say(f"stepped rows {rows} x {cols}")
    assert bit_equal(H.add(a2, d, alpha=0.5), oracle.add(a2, d, alpha=0.5))
    assert bit_equal(H.add(d, a2), oracle.add(d, a2))
    assert bit_equal(H.add(a3, d, alpha=-2.0), oracle.add(a3, d, alpha=-2.0))
    assert bit_equal(H.add(d, a3), oracle.add(d, a3))
    assert bit_equal(H.add(a2, x2[:, 1::2]), oracle.add(a2, x2[:, 1::2]))         # second input unaligned
    assert bit_equal(H.add(a2, a3, alpha=0.25), oracle.add(a2, a3, alpha=0.25))
    assert bit_equal(H.add(a3, a2), oracle.add(a3, a2))
    assert bit_equal(H.add(a2, a2), oracle.add(a2, a2))
    assert bit_equal(H.add(a3, x3[:, 2::3]), oracle.add(a3, x3[:, 2::3]))         # ends with the storage
    assert bit_equal(H.binary("twg_mul_f32", a3, d), a3 * d)
    assert bit_equal(H.unary("twg_unary_f32", a2, pre=(ctypes.c_int(1),)), torch.relu(a2))
    assert bit_equal(H.unary("twg_unary_f32", a3, pre=(ctypes.c_int(0),)), a3.contiguous())
    # rows that do not merge (a narrower view of the stepped rows), and three dimensions
    w = cols - 4
    assert bit_equal(H.add(a2[:, :w], d[:, :w]), oracle.add(a2[:, :w], d[:, :w]))
    assert bit_equal(H.add(a3[:, 4:], d[:, 4:]), oracle.add(a3[:, 4:], d[:, 4:]))
    y = torch.randn(3, rows, 2 * cols, generator=g)
    e = torch.randn(3, rows, cols, generator=g)
    assert bit_equal(H.add(y[..., ::2], e), oracle.add(y[..., ::2], e))
    assert bit_equal(H.add(y[1:, :, ::2], e[0]), oracle.add(y[1:, :, ::2], e[0]))  # e read again
    assert bit_equal(H.add(y.transpose(0, 1)[..., ::2], e.transpose(0, 1)),
                     oracle.add(y.transpose(0, 1)[..., ::2], e.transpose(0, 1)))
    # output stepped as well stays with the general walk
    o = torch.zeros(rows, 2 * cols)[:, ::2]
    assert bit_equal(H.add(a2, d, out=o), oracle.add(a2, d))


@pytest.mark.parametrize("rows,cols,pad,start", [
    (37, 1000, 1, 1), (37, 1000, 5, 0), (50, 1001, 3, 2), (9, 4099, 1, 1), (300, 256, 2, 1),
    (3, 70001, 7, 3), (64, 999, 0, 0), (130, 66, 1, 1)])
def test_rows_that_start_anywhere(twg, rows, cols, pad, start):
    # x[:, 1:], a row pitch that is not a multiple of 4 elements, rows whose length is not one:
    # the row kernel moves 16-byte packs at 4-byte alignment and finishes each row element by
    # element.  One or both inputs sliced, the output contiguous or sliced as well, a bias row,
    # and activations over the same views.
    import twg_capi as C
    g = torch.Generator().manual_seed(rows * cols + pad)
    big_a = torch.randn(rows, cols + pad, generator=g)
    big_b = torch.randn(rows, cols + pad, generator=g)
    a = big_a[:, start:start + cols]
    b = big_b[:, start:start + cols]
    bc = torch.randn(rows, cols, generator=g)
    assert bit_equal(H.add(a, bc, alpha=0.5), oracle.add(a, bc, alpha=0.5))
    assert bit_equal(H.add(bc, a), oracle.add(bc, a))
    assert bit_equal(H.add(a, b, alpha=-1.5), oracle.add(a, b, alpha=-1.5))
    out = torch.zeros(rows, cols + pad)[:, start:start + cols]
    assert bit_equal(H.add(a, b, out=out), oracle.add(a, b))
    bias = torch.randn(1, cols + pad, generator=g)[:, start:start + cols]
    assert bit_equal(H.add(a, bias), oracle.add(a, bias))
    col = torch.randn(rows, 1, generator=g)
    assert bit_equal(H.add(a, col), oracle.add(a, col))
    assert bit_equal(_unary(C.UNARY_RELU, a), torch.relu(a))
    got = _unary(C.UNARY_GELU_ERF, a)
    assert rel_err_ok(got, closed_form64("gelu_erf", a))[0]
    assert bit_equal(H.binary("twg_eq_f32", a, b, out_dtype=torch.bool), torch.eq(a, b))
    # compares over the same rows: four bools per lane, into an aligned and a shifted output
    z = torch.where(torch.rand(rows, cols + pad, generator=g) < 0.3, torch.zeros(()), big_a)[:, start:start + cols]
    assert bit_equal(H.unary("twg_ne_scalar_f32", z, out_dtype=torch.bool, extra=(ctypes.c_float(0.0),)), z.ne(0.0))
    mout = torch.zeros(rows, cols + pad, dtype=torch.bool)[:, start:start + cols]
    assert bit_equal(H.binary("twg_eq_f32", a, b, out=mout), torch.eq(a, b))


def test_outputs_that_no_input_streams_into(twg):
    # outer sums and doubly broadcast operands: both inputs are re-read from cache and a block
    # only streams its store (four packs per lane there); rows from 1024 elements on, with a
    # ragged length, misaligned, and too short for that path
    g = torch.Generator().manual_seed(77)
    for n, m in ((300, 4096), (257, 4100), (64, 1024), (33, 5001), (70, 1000)):
        col, row = torch.randn(n, 1, generator=g), torch.randn(1, m, generator=g)
        assert bit_equal(H.add(col, row, alpha=1.25), oracle.add(col, row, alpha=1.25)), (n, m)
        assert bit_equal(H.add(row, col), oracle.add(row, col)), (n, m)
        rowv = torch.randn(1, m + 3, generator=g)[:, 1:m + 1]
        assert bit_equal(H.add(col, rowv), oracle.add(col, rowv)), (n, m)
    a = torch.randn(37, 1, 2048, generator=g)
    b = torch.randn(1, 19, 2048, generator=g)
    assert bit_equal(H.add(a, b), oracle.add(a, b))
    # the same geometry whatever order the dimensions are passed in: a transposed output with
    # transposed inputs, all in logical order (no sorting by output stride on the caller's side)
    x, y = torch.randn(130, 515, generator=g).t(), torch.randn(130, 515, generator=g).t()
    out = torch.zeros(130, 515).t()
    got = H.binary("twg_add_f32", x, y, out=out, extra=(ctypes.c_float(1.0),), sort_by_out=False)
    assert bit_equal(got, x + y)
    nhwc = torch.randn(3, 20, 20, 64, generator=g).permute(0, 3, 1, 2)
    bias = torch.randn(1, 64, 1, 1, generator=g)
    out = torch.zeros(3, 20, 20, 64).permute(0, 3, 1, 2)
    got = H.binary("twg_add_f32", nhwc, bias, out=out, extra=(ctypes.c_float(1.0),), sort_by_out=False)
    assert bit_equal(got, nhwc + bias)


def test_add_generic_strides_bruteforce(twg):
    g = torch.Generator().manual_seed(5)
    sizes = [3, 4, 2, 5]
    for perm in itertools.permutations(range(4)):
        a = torch.randn(*sizes, generator=g).permute(*perm)
        for bc in (0, 1, 6, 9, 15):
            bshape = [1 if (bc >> d) & 1 else a.shape[d] for d in range(4)]
            b = torch.randn(11 + int(torch.tensor(bshape).prod()), generator=g)[11:].view(*bshape)
            ref = oracle.add(a, b, alpha=1.5)
            assert bit_equal(H.add(a, b, alpha=1.5), ref)
            # keep the logical dimension order too (no sorting by output stride)
            assert bit_equal(H.binary("twg_add_f32", a, b, extra=(ctypes.c_float(1.5),),
                                      sort_by_out=False), ref)
    # 8 dimensions, negative stride via flip is not expressible in torch; use steps
    a8 = torch.randn(2, 3, 2, 2, 3, 2, 2, 3, generator=g)[:, ::2, :, :, ::2]
    b8 = torch.randn(2, 1, 2, 1, 1, 2, 1, 3, generator=g)
    assert bit_equal(H.add(a8, b8), a8 + b8)


def _random_view(g, shape, rng):
    """A tensor of logical `shape` with random memory layout: permuted dimensions,
    stepped slices, a storage offset of 0..3 elements."""
    nd = len(shape)
    perm = rng.sample(range(nd), nd)
    steps = [rng.choice((1, 1, 1, 2, 3)) for _ in range(nd)]
    phys = [shape[perm[i]] * steps[perm[i]] for i in range(nd)]
    off = rng.randrange(4)
    numel = 1
    for e in phys:
        numel *= e
    base = torch.randint(-8, 8, (numel + off,), generator=g).float()[off:].view(*phys)
    inv = [perm.index(d) for d in range(nd)]
    t = base.permute(*inv)
    return t[tuple(slice(None, None, steps[d]) for d in range(nd))]


def test_random_strips_and_ragged_rows(twg):
    # Seeded shapes aimed at two launch paths whose index arithmetic depends on the extents:
    # an operand stored [.., x, c] with 2..31 channels against a [.., c, x] output (strips
    # through LDS: one strip per block, several strips of short rows per block, last strips that
    # are shorter, channel counts that do and do not divide the LDS pitch), the mirror image of
    # that (planar operand, [.., x, c] output), and rows whose
    # starts fall anywhere into the output's 128-byte lines (chunks cut at those lines).
    import random
    rng = random.Random(4321)
    g = torch.Generator().manual_seed(99)
    for case in range(48):
        c = rng.choice((2, 3, 4, 5, 7, 8, 12, 16, 17, 24, 31))
        x = rng.choice((32, 40, 96, 100, 224, 256, 260, 513, 1024, 1500, 4099))
        outer = rng.choice(((2,), (3,), (2, 3), (5, 2)))
        while torch.Size(outer).numel() * c * x > (1 << 19):
            x = max(32, x // 2)
        off = rng.choice((0, 0, 1, 4))
        stored = torch.randn(off + torch.Size(outer).numel() * x * c, generator=g)[off:].view(*outer, x, c)
        a = stored.transpose(-1, -2)                     # logical [.., c, x], unit stride along c
        b = torch.randn(*outer, c, x, generator=g)
        _say(f"strip case {case}: {tuple(a.shape)} stored {tuple(stored.shape)} offset {off}")
        assert bit_equal(H.add(a, b, alpha=0.5), oracle.add(a, b, alpha=0.5))
        assert bit_equal(H.add(b, a), oracle.add(b, a))
        stored2 = torch.randn(*outer, x, c, generator=g)
        assert bit_equal(H.add(a, stored2.transpose(-1, -2)), oracle.add(a, stored2.transpose(-1, -2)))
        # the mirror image: output [.., x, c], operand stored planar [.., c, x]
        planar = torch.randn(off + torch.Size(outer).numel() * x * c, generator=g)[off:].view(*outer, c, x)
        pa = planar.transpose(-1, -2)                    # logical [.., x, c], unit stride along x
        assert bit_equal(H.add(pa, stored2, alpha=0.25), oracle.add(pa, stored2, alpha=0.25))
        assert bit_equal(H.add(stored2, pa), oracle.add(stored2, pa))
        assert bit_equal(H.add(pa, b.transpose(-1, -2)), oracle.add(pa, b.transpose(-1, -2)))
        assert bit_equal(H.unary("twg_unary_f32", pa, pre=(ctypes.c_int(1),)), torch.relu(pa))
    for case in range(32):
        rows = rng.choice((3, 17, 64, 200))
        # three chunks and more; from 8192 elements on the row kernel takes them, below that the pack walk
        length = 4 * rng.choice((193, 250, 251, 300, 511, 1000, 2047, 2050, 2051, 2251, 3073))
        lead = rng.choice((0, 4, 8, 20, 28))                                    # row 0 starts here
        pitch = length + 4 * rng.choice((0, 1, 2, 3, 5, 8))
        big_o = torch.zeros(lead + rows * pitch)
        out = big_o[lead:].as_strided((rows, length), (pitch, 1))
        big_a = torch.randn(lead + rows * pitch, generator=g)
        a = big_a[lead:].as_strided((rows, length), (pitch, 1))
        colv = torch.randn(rows, 1, generator=g)
        full = torch.randn(rows, length, generator=g)
        _say(f"ragged rows {case}: {rows} x {length}, pitch {pitch}, lead {lead}")
        assert bit_equal(H.add(a, colv, out=out), oracle.add(a, colv))
        assert bool((big_o[:lead] == 0).all())
        if pitch > length:
            gaps = big_o[lead:].as_strided((rows - 1, pitch - length), (pitch, 1), length)
            assert bool((gaps == 0).all()), "wrote between the rows"
        assert bit_equal(H.add(full, colv), oracle.add(full, colv))
        assert bit_equal(H.add(a, full), oracle.add(a, full))


def test_random_geometries(twg):
    # 120 seeded layouts: every dispatch path of the elementwise launcher (contiguous,
    # rows with broadcast operands, LDS tiles, 128-bit tiles, div/mod) and the strided
    # masked_select, against ATen's CPU kernels on the very same views.  (The same loop ran
    # for ~15000 layouts with other seeds without a difference.)
    import random
    rng = random.Random(1234)
    g = torch.Generator().manual_seed(77)
    extents = (1, 2, 3, 4, 5, 8, 16, 63, 64, 65, 128, 260)
    for case in range(120):
        nd = rng.randint(1, 5)
        shape = [rng.choice(extents) for _ in range(nd)]
        while torch.Size(shape).numel() > (1 << 18):
            shape[rng.randrange(nd)] = rng.choice(extents[:6])
        bshape = [1 if rng.random() < 0.3 else e for e in shape]
        ashape = list(shape) if rng.random() < 0.8 else [1 if rng.random() < 0.3 else e for e in shape]
        a, b = _random_view(g, ashape, rng), _random_view(g, bshape, rng)
        _say(f"geometry {case}: a {tuple(a.shape)}/{a.stride()} b {tuple(b.shape)}/{b.stride()}")
        assert bit_equal(H.add(a, b), a + b)
        out = _random_view(g, list(torch.broadcast_shapes(a.shape, b.shape)), rng)
        assert bit_equal(H.add(a, b, alpha=-2.0, out=out), a + b * -2.0)  # small integers: exact
        eq = H.binary("twg_eq_f32", a, b, out_dtype=torch.bool)
        assert torch.equal(eq, torch.eq(a, b))
        if case % 3 == 0:
            vals, k = H.masked_select(a, torch.eq(a, b))
            ref = torch.masked_select(a, torch.eq(a, b))
            assert k == ref.numel() and bit_equal(vals, ref)
        # the same layouts in another dtype: compare, compaction and conversion
        dt = (torch.int64, torch.float16, torch.uint8, torch.bool, torch.float64)[case % 5]

        def relayout(t, like):
            return torch.empty_strided(like.shape, like.stride(), dtype=t.dtype).copy_(t)

        ad = relayout(a > 0 if dt == torch.bool else a.to(dt), a)
        bd = relayout(b > 0 if dt == torch.bool else b.to(dt), b)
        assert torch.equal(H.compare_eq(ad, bd), torch.eq(ad, bd)), dt
        vals, k = H.masked_select(ad, a > 0)
        assert bit_equal(vals, torch.masked_select(ad, a > 0)), dt
        rc, got = H.cast(ad, torch.float32)
        assert rc == 0 and bit_equal(got, ad.to(torch.float32)), dt


def test_short_rows_with_a_small_broadcast_operand(twg):
    # [rows, len] with len below one block's span plus a row vector or a per-row value on
    # either side of a non-commutative form: the flat kernel, and its fallbacks when the row
    # length is not a multiple of 4 or a pointer is misaligned
    g = torch.Generator().manual_seed(41)
    for rows, ln in ((1000, 4), (333, 8), (4097, 16), (70, 60), (5000, 64), (257, 100), (300, 252),
                     (129, 62), (64, 256), (1001, 5), (77, 63), (401, 10), (3, 7), (50, 3), (1, 9),
                     (37, 320), (9, 1001), (5, 4092), (3, 4096), (2, 5000)):
        _say(f"short rows {rows}x{ln}")
        big = torch.randn(rows, ln, generator=g)
        rowv = torch.randn(ln, generator=g)
        colv = torch.randn(rows, 1, generator=g)
        for small in (rowv, colv, colv[::2].repeat_interleave(2, 0)[:rows], torch.randn(1, 1, generator=g)):
            assert bit_equal(H.add(big, small, alpha=-2.5), oracle.add(big, small.expand_as(big), alpha=-2.5))
            assert bit_equal(H.add(small, big, alpha=-2.5), oracle.add(small.expand_as(big), big, alpha=-2.5))
            assert torch.equal(H.binary("twg_eq_f32", big, small, out_dtype=torch.bool), torch.eq(big, small))
        # a strided per-row operand (every third value of a longer vector)
        col3 = torch.randn(3 * rows, generator=g)[::3].unsqueeze(1)
        assert bit_equal(H.binary("twg_mul_f32", big, col3), big * col3)
        # misaligned dense operand and misaligned row vector
        flat = torch.randn(rows * ln + 1, generator=g)
        big1 = flat[1:].view(rows, ln)
        assert bit_equal(H.add(big1, rowv), big1 + rowv)
        rowv1 = torch.randn(ln + 1, generator=g)[1:]
        assert bit_equal(H.add(big, rowv1), big + rowv1)


def test_short_unit_stride_rows_in_strided_arrangements(twg):
    # rows of 32..252 elements that are unit-stride (or broadcast) in every operand but laid
    # out with gaps, permuted outer dimensions or mixed broadcasts: the packed general kernel,
    # and the element-wise one where a pack would be misaligned
    g = torch.Generator().manual_seed(43)
    base = torch.randn(40, 6, 8, 128, generator=g)
    other = torch.randn(40, 8, 6, 64, generator=g)
    x = base[..., :64]                       # sliced rows
    y = other.permute(0, 2, 1, 3)            # permuted outer dimensions
    for a, b in ((x, y), (y, x), (x, x[:, :1]), (x[:, :, :1], y), (x, torch.randn(64, generator=g)),
                 (base[..., 32:96], y), (base[..., 4:68], y), (base[..., 1:65], y)):
        assert bit_equal(H.add(a, b, alpha=0.75), oracle.add(a.expand(40, 6, 8, 64), b.expand(40, 6, 8, 64), alpha=0.75))
        assert torch.equal(H.binary("twg_eq_f32", a, b, out_dtype=torch.bool), torch.eq(a, b))
        out = torch.zeros(40, 6, 8, 96)[..., 16:80]
        assert bit_equal(H.add(a, b, out=out), a + b)
    import twg_capi as C
    assert bit_equal(H.unary("twg_unary_f32", x, pre=(C.UNARY_RELU,)), torch.relu(x))
    got = H.unary("twg_unary_f32", y, pre=(C.UNARY_GELU_ERF,), out=torch.zeros(40, 6, 8, 128)[..., 64:])
    assert rel_err_ok(got, closed_form64("gelu_erf", y))[0]
    for ln in (32, 36, 100, 252):
        z = torch.randn(300, 256, generator=g)[:, :ln]
        w = torch.randn(300, 1, generator=g)
        assert bit_equal(H.binary("twg_mul_f32", z, w), z * w)
        assert bit_equal(H.binary("twg_mul_f32", w, z), w * z)


def test_dense_operand_with_gathered_small_operand(twg):
    # output and one input dense, the other broadcast or strided over up to four dimensions
    # with short or ragged rows (a channel bias over [N, C, 7, 7] and the like): the flat
    # kernel that gathers the small operand, on either side of a non-commutative form
    g = torch.Generator().manual_seed(47)
    for shape in ((9, 10, 7, 7), (6, 5, 3, 27), (33, 81), (4, 7, 9, 5), (5, 3, 2, 2), (2, 300, 3)):
        big = torch.randn(*shape, generator=g)
        nd = len(shape)
        for keep in itertools.product((True, False), repeat=nd):
            if all(keep):
                continue
            small = torch.randn(*[s if k else 1 for s, k in zip(shape, keep)], generator=g)
            _say(f"gathered operand {shape} + {tuple(small.shape)}")
            assert bit_equal(H.add(big, small, alpha=1.5), oracle.add(big, small.expand(shape), alpha=1.5))
            assert bit_equal(H.add(small, big, alpha=1.5), oracle.add(small.expand(shape), big, alpha=1.5))
            assert torch.equal(H.binary("twg_eq_f32", small, big, out_dtype=torch.bool), torch.eq(small, big))
        # a strided (not broadcast) small side: every other element of a wider tensor
        wide = torch.randn(*shape[:-1], 2 * shape[-1], generator=g)
        assert bit_equal(H.binary("twg_mul_f32", big, wide[..., ::2]), big * wide[..., ::2])
        assert bit_equal(H.binary("twg_mul_f32", wide[..., 1::2], big), wide[..., 1::2] * big)


def test_mul_and_fused_add_relu(twg):
    g = torch.Generator().manual_seed(6)
    a = torch.randn(70001, generator=g)
    b = torch.randn(70001, generator=g)
    assert bit_equal(H.binary("twg_mul_f32", a, b), oracle.mul(a, b))
    assert bit_equal(H.binary("twg_add_relu_f32", a, b), oracle.add_relu(a, b))
    # reference vectors: tests/ops/test_mul.py:30-39, tests/test_dev.py:8-18
    assert torch.equal(H.binary("twg_mul_f32", torch.tensor([[1., 2.], [3., 4.]]),
                                torch.tensor([10., 20.])),
                       torch.tensor([[10., 40.], [30., 80.]]))
    r = H.binary("twg_add_relu_f32", torch.tensor([-1.5, 2.7, 1.0, 2.0]),
                 torch.tensor([-1.0, 0.9, 1.1, -2.1]))
    assert torch.allclose(r, torch.tensor([0, 3.6, 2.1, 0]))
    s = H.unary("twg_add_scalar_f32", a, extra=(ctypes.c_float(2.5), ctypes.c_float(0.5)))
    assert bit_equal(s, oracle.add(a, torch.full_like(a, 2.5), alpha=0.5))
    m = H.unary("twg_mul_scalar_f32", a, extra=(ctypes.c_float(2.0),))
    assert bit_equal(m, a * 2.0)


# ------------------------------------------------------------------- casts

_INT_TYPES = (torch.bool, torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64)
_FLOAT_TYPES = (torch.float16, torch.bfloat16, torch.float32, torch.float64)


def _cast_source(dtype, n, g):
    """Values every target type can hold (0..100 plus specials that stay defined)."""
    if dtype == torch.bool:
        return torch.rand(n, generator=g) < 0.5
    if dtype in _INT_TYPES:
        t = torch.randint(0, 101, (n,), generator=g).to(dtype)
        if dtype == torch.int64:  # beyond 2^24 and 2^53: rounding on the way to float
            t[:6] = torch.tensor([16777217, 33554435, (1 << 53) + 1, 123456789012345, 0, 1])
        return t
    t = (torch.rand(n, generator=g, dtype=torch.float64) * 100).to(dtype)
    t[:8] = torch.tensor([0.0, -0.0, 0.5, 0.999, 1.5, 2.5, 99.99, 3.0]).to(dtype)
    return t


def test_cast_direct_pairs_match_aten(twg):
    # every direct pair of twg_cast against ATen's CPU conversion of the same values
    g = torch.Generator().manual_seed(21)
    L = twg.load()
    n = 70001
    direct = 0
    for src_t in _INT_TYPES + _FLOAT_TYPES:
        for dst_t in _INT_TYPES + _FLOAT_TYPES:
            if src_t == dst_t:
                continue
            a = _cast_source(src_t, n, g)
            rc, got = H.cast(a, dst_t)
            if rc == twg.E_UNSUPPORTED:
                continue
            twg.check(rc)
            direct += 1
            _say(f"cast {src_t} -> {dst_t}")
            assert bit_equal(got, a.to(dst_t)), (src_t, dst_t)
            # misaligned base pointers and a strided source / destination (div/mod kernel)
            rc, got = H.cast(a[1:], dst_t)
            assert rc == 0 and bit_equal(got, a[1:].to(dst_t))
            a2 = a[:60000].view(200, 300).t()
            rc, got = H.cast(a2, dst_t, out=torch.zeros(300, 400, dtype=dst_t)[:, ::2])
            assert rc == 0 and bit_equal(got, a2.to(dst_t))
    assert direct == 31
    assert L.twg_cast(None, 99, None, 0, None, None) == twg.E_INVALID_ARG


def test_cast_float_edge_cases(twg):
    # rounding to half / bfloat16 (ties, overflow to inf, subnormals), NaN and inf,
    # float -> bool on values that vanish in a narrower type, negative truncation
    f = torch.tensor([1.0 + 2 ** -11, 1.0 + 3 * 2 ** -11, 65504.0, 65520.0, 65519.99, 1e-8, 6e-8,
                      -6.1e-5, float("inf"), -float("inf"), float("nan"), 3.3895314e38,
                      1.0 + 2 ** -8, 1.0 + 3 * 2 ** -8, 1e-40, -1e-45, 0.0, -0.0])
    for dst_t in (torch.float16, torch.bfloat16, torch.float64, torch.bool):
        rc, got = H.cast(f, dst_t)
        ref = f.to(dst_t)
        assert rc == 0
        assert bit_equal(got, ref) or (dst_t != torch.bool and torch.equal(got.isnan(), ref.isnan())
                                       and bit_equal(got.nan_to_num(), ref.nan_to_num()))
    d = torch.tensor([1e-300, -1e-310, 0.0, -0.0, float("nan"), 1e300, 16777217.0, 0.1],
                     dtype=torch.float64)
    rc, got = H.cast(d, torch.bool)
    assert rc == 0 and torch.equal(got, d.to(torch.bool))
    rc, got = H.cast(d, torch.float32)
    assert rc == 0 and bit_equal(got.nan_to_num(), d.to(torch.float32).nan_to_num())
    neg = torch.tensor([-0.9, -1.0, -1.5, -2.5, -100.7, 100.7, 2147483000.0, -2147483000.0])
    for dst_t in (torch.int32, torch.int64, torch.int16, torch.int8):
        src = neg if dst_t in (torch.int32, torch.int64) else neg[:6]
        rc, got = H.cast(src, dst_t)
        assert rc == 0 and torch.equal(got, src.to(dst_t)), dst_t
    for src_t in (torch.float16, torch.bfloat16):
        h = f.to(src_t)
        rc, got = H.cast(h, torch.float32)
        assert rc == 0 and bit_equal(got.nan_to_num(), h.to(torch.float32).nan_to_num())


def _compare_source(dtype, n, g):
    """Few distinct values (so that about a fifth of the pairs match) plus the type's specials."""
    if dtype == torch.bool:
        return torch.rand(n, generator=g) < 0.5
    if dtype in _INT_TYPES:
        info = torch.iinfo(dtype)
        t = torch.randint(0, 5, (n,), generator=g).to(dtype)
        t[:4] = torch.tensor([info.min, info.max, info.min, 0], dtype=dtype)
        return t
    t = torch.randint(-2, 3, (n,), generator=g).to(dtype)
    t[:8] = torch.tensor([0.0, -0.0, float("nan"), float("inf"), -float("inf"), 0.5, 1.0, -1.0]).to(dtype)
    return t


def test_eq_ne_and_every_dtype_match_aten(twg):
    # twg_eq / twg_ne_scalar / twg_and against ATen's CPU kernels: dense, misaligned,
    # broadcast and strided operands of every dtype
    g = torch.Generator().manual_seed(33)
    n = 50021
    for dt in _INT_TYPES + _FLOAT_TYPES:
        _say(f"eq/ne/and {dt}")
        a, b = _compare_source(dt, n, g), _compare_source(dt, n, g)
        b[:8] = a[:8].flip(0)  # specials against specials: NaN vs NaN, 0.0 vs -0.0, min vs max
        b[8:16] = a[8:16]
        assert torch.equal(H.compare_eq(a, b), torch.eq(a, b)), dt
        assert torch.equal(H.compare_eq(a[1:], b[:-1]), torch.eq(a[1:], b[:-1])), dt
        a2, row = a[:50000].view(250, 200), b[:200]
        assert torch.equal(H.compare_eq(a2, row), torch.eq(a2, row)), dt
        assert torch.equal(H.compare_eq(a2.t(), b[21:50021].view(200, 250)),
                           torch.eq(a2.t(), b[21:50021].view(200, 250))), dt
        if dt in _FLOAT_TYPES:
            for s in (0.0, 1.0, 0.1, float("nan"), float("inf"), 1.0 + 2 ** -12):
                # the reference value: ATen rounds the scalar to the tensor's dtype
                assert torch.equal(H.compare_ne_scalar(a, s, 0), a.ne(s)), (dt, s)
        elif dt == torch.bool:
            for s in (0, 1):
                assert torch.equal(H.compare_ne_scalar(a, 0.0, s), a.ne(bool(s))), (dt, s)
        else:
            info = torch.iinfo(dt)
            for s in (0, 3, info.max, info.min):
                assert torch.equal(H.compare_ne_scalar(a, 0.0, s), a.ne(s)), (dt, s)
            assert torch.equal(H.compare_ne_scalar(a2.t(), 0.0, 3), a2.t().ne(3)), dt
        if dt in _INT_TYPES:
            x = _compare_source(dt, n, g)
            if dt not in (torch.bool,):
                x = torch.randint(0, 1 << 7, (n,), generator=g).to(dt) * (3 if dt != torch.int8 else 1)
            y = x.flip(0).clone()
            assert bit_equal(H.bitwise_and(x, y), torch.bitwise_and(x, y)), dt
            assert bit_equal(H.bitwise_and(x[:50000].view(250, 200).t(), y[:250]),
                             torch.bitwise_and(x[:50000].view(250, 200).t(), y[:250])), dt
    # abs: every dtype but bool; integers wrap at their minimum, NaN and -0.0 lose their sign
    for dt in _INT_TYPES + _FLOAT_TYPES:
        a = _compare_source(dt, n, g)
        if dt in _FLOAT_TYPES:
            a = -a
        elif dt not in (torch.bool, torch.uint8):
            a = a - 2
            a[0] = torch.iinfo(dt).min
        rc, got = H.abs_any(a)
        if dt == torch.bool:
            assert rc == twg.E_UNSUPPORTED
            continue
        assert rc == 0 and bit_equal(got, a.abs()), dt
        rc, got = H.abs_any(a[:50000].view(250, 200).t(), out=torch.zeros(200, 500, dtype=dt)[:, ::2])
        assert rc == 0 and bit_equal(got, a[:50000].view(250, 200).t().abs()), dt
    L = twg.load()
    assert L.twg_eq(None, None, None, 99, None, None) == twg.E_INVALID_ARG
    assert L.twg_and(None, None, None, 3, None, None) == twg.E_UNSUPPORTED


@pytest.mark.parametrize("dtype", [torch.bool, torch.uint8, torch.int16, torch.float16, torch.bfloat16,
                                   torch.int32, torch.int64, torch.float64])
def test_masked_select_every_element_size(twg, dtype):
    # elements are moved, not looked at: 1, 2, 4 and 8 bytes, dense, misaligned, broadcast, strided
    g = torch.Generator().manual_seed(34)
    for n in (1, 63, 4096, 70001, (1 << 21) + 5):
        _say(f"masked_select {dtype} n={n}")
        x = (torch.randn(n, generator=g) * 1000).to(dtype)
        m = torch.rand(n, generator=g) < 0.4
        vals, k = H.masked_select(x, m, check_guard=True)
        assert k == int(m.sum()) and bit_equal(vals, torch.masked_select(x, m)), (dtype, n)
    x = (torch.randn(40004, generator=g) * 1000).to(dtype)
    m = torch.rand(40004, generator=g) < 0.5
    vals, _ = H.masked_select(x[1:40001], m[3:40003], out_offset=1, check_guard=True)
    assert bit_equal(vals, torch.masked_select(x[1:40001], m[3:40003]))
    xt = x[:40000].view(100, 400).t()
    vals, _ = H.masked_select(xt, m[:100])
    assert bit_equal(vals, torch.masked_select(xt, m[:100]))


@pytest.mark.parametrize("dtype", [torch.uint8, torch.int16, torch.int64, torch.float64])
def test_masked_select_fast_kernels_every_element_size(twg, dtype):
    # the streaming kernel (all three tile sizes, with an incomplete last tile) and the tile variant
    # for 1-, 2- and 8-byte elements: dense and sparse masks, runs, shifted output pointers
    g = torch.Generator().manual_seed(35)
    es = torch.empty(0, dtype=dtype).element_size()
    for n in (8192 * 3 + 17, (1 << 21) + 8192 + 5, (1 << 23) + 70001, (1 << 25) + 131072 + 4099):
        if dtype.is_floating_point:
            x = torch.randn(n, generator=g, dtype=dtype)
        else:
            info = torch.iinfo(dtype)
            x = torch.randint(max(info.min, -(1 << 62)), min(info.max, 1 << 62), (n,), generator=g,
                              dtype=dtype)
        idx = torch.arange(n)
        masks = {
            "p=0.5": torch.rand(n, generator=g) < 0.5,
            "p=0.99": torch.rand(n, generator=g) < 0.99,
            "p=0.02": torch.rand(n, generator=g) < 0.02,
            "every 16th": idx % 16 == 5,
            "runs": (idx % 5003) < 2500,
            "last only": idx == n - 1,
        }
        for name, m in masks.items():
            ref = torch.masked_select(x, m)
            for off in (0, 1, 128 // es - 1):
                _say(f"masked_select {dtype} n={n} {name} out_offset={off}")
                vals, k = H.masked_select(x, m, out_offset=off, check_guard=True)
                assert k == ref.numel() and bit_equal(vals, ref), (dtype, n, name, off)


# ------------------------------------------------------------- activations

def _unary(op, x, **kw):
    return H.unary("twg_unary_f32", x, pre=(ctypes.c_int(op),), **kw)


def test_relu_and_copy_bits(twg):
    import twg_capi as C
    x = W.activation_input(512, 1024, seed=1)
    assert bit_equal(_unary(C.UNARY_RELU, x), oracle.relu(x))
    assert bit_equal(_unary(C.UNARY_RELU, x), torch.relu(x))
    assert bit_equal(_unary(C.UNARY_COPY, x), x)
    assert bit_equal(_unary(C.UNARY_ABS, x), oracle.unary(oracle.ABS, x))
    s = torch.tensor([-0.0, 0.0, -1.0, 1.0, float("nan"), float("inf"), -float("inf"), -1e-45,
                      1e-45, 1e-30, -1e-30])
    got = _unary(C.UNARY_RELU, s)
    assert ulp_diff(got, torch.relu(s)) == 0
    assert torch.equal(torch.signbit(got), torch.signbit(torch.relu(s)))
    # strided input, transposed output
    xt = x.t()
    assert bit_equal(_unary(C.UNARY_RELU, xt), torch.relu(xt))
    assert bit_equal(_unary(C.UNARY_COPY, xt), xt.contiguous())
    assert bit_equal(_unary(C.UNARY_COPY, x[::3, 5:900:7]), x[::3, 5:900:7].contiguous())


@pytest.mark.parametrize("name", ["gelu_erf", "gelu_tanh", "silu"])
def test_activation_golden_points(twg, name):
    import twg_capi as C
    op = {"gelu_erf": C.UNARY_GELU_ERF, "gelu_tanh": C.UNARY_GELU_TANH, "silu": C.UNARY_SILU}[name]
    x, ref = load_activation_golden()
    got = _unary(op, x)
    ok, err, bound = rel_err_ok(got, ref[name], floor=FLOOR[name])
    worst = int(torch.argmax(err / bound))
    assert ok, f"{name}: x={x[worst].item()!r} got={got[worst].item()!r} ref={ref[name][worst].item()!r}"
    # signed zeros and tiny inputs, as ATen's CPU kernels give them
    z = torch.tensor([0.0, -0.0, 1e-30, -1e-30])
    gz = _unary(op, z)
    assert torch.equal(torch.signbit(gz), torch.tensor([False, True, False, True]))
    assert bool((gz[:2] == 0).all())
    assert rel_err_ok(gz[2:], torch.tensor([5.000000015855384e-31, -5.000000015855384e-31],
                                            dtype=torch.float64))[0]
    # NaN propagates, +inf -> +inf
    s = _unary(op, torch.tensor([float("nan"), float("inf")]))
    assert torch.isnan(s[0]) and s[1] == float("inf")


@pytest.mark.parametrize("name", ["gelu_erf", "gelu_tanh", "silu"])
def test_activation_config2_distribution(twg, name):
    import twg_capi as C
    op = {"gelu_erf": C.UNARY_GELU_ERF, "gelu_tanh": C.UNARY_GELU_TANH, "silu": C.UNARY_SILU}[name]
    x = W.activation_input(1024, 2048, seed=1)  # N(0, 9) with forced 0 / +-1e-30 entries
    # widen the tails beyond what 2^21 samples reach: 2^28 samples reach |x| ~ 18.7
    x.view(-1)[:4096] = torch.linspace(-19.0, 19.0, 4096)
    got = _unary(op, x)
    ref64 = closed_form64(name, x)
    ok, err, bound = rel_err_ok(got, ref64, floor=FLOOR[name])
    worst = int(torch.argmax((err / bound).view(-1)))
    assert ok, f"{name}: x={x.view(-1)[worst].item()!r} err={err.view(-1)[worst].item()}"
    # the oracle (closed form rounded once) agrees to the same bar
    ora = oracle.unary({"gelu_erf": oracle.GELU_ERF, "gelu_tanh": oracle.GELU_TANH,
                        "silu": oracle.SILU}[name], x)
    ok2, _, _ = rel_err_ok(got, ora.double(), floor=FLOOR[name])
    assert ok2
    # ATen's CPU kernels, at the tolerances the reference's own tests use
    if name == "silu":
        assert torch.allclose(got, F.silu(x), atol=1e-6)   # tests/ops/test_silu.py:13
    else:
        assert torch.allclose(got, F.gelu(x), atol=1e-3)   # tests/ops/test_gelu.py:14
    if name == "gelu_erf":
        assert torch.allclose(got, F.gelu(x), atol=2e-6, rtol=0)


def test_activation_reference_vectors(twg):
    import twg_capi as C
    for data in ([-1.0, 0.0, 1.0, 2.0], [[0.5, -0.5], [1.5, -1.5]], [2.0], [0.0]):
        t = torch.tensor(data, dtype=torch.float32)
        assert torch.allclose(_unary(C.UNARY_GELU_ERF, t), F.gelu(t), atol=1e-3)
        assert torch.allclose(_unary(C.UNARY_GELU_TANH, t), F.gelu(t), atol=1e-3)
        assert torch.allclose(_unary(C.UNARY_SILU, t), F.silu(t), atol=1e-6)


# ------------------------------------------------------------------- masks

def test_mask_ops_config4(twg):
    n = (1 << 20) + 5
    p, q, z = W.mask_inputs(n, seed=3)
    e = H.binary("twg_eq_f32", p, q, out_dtype=torch.bool)
    assert e.dtype == torch.bool and bit_equal(e, oracle.eq(p, q)) and bit_equal(e, torch.eq(p, q))
    assert 0.05 < e.float().mean().item() < 0.075  # about 1/16
    nz = H.unary("twg_ne_scalar_f32", z, out_dtype=torch.bool, extra=(ctypes.c_float(0.0),))
    assert bit_equal(nz, oracle.ne_scalar(z, 0.0)) and bit_equal(nz, z.ne(0.0))
    assert 0.69 < nz.float().mean().item() < 0.71
    both = H.binary("twg_and_u8", e, nz, out_dtype=torch.bool)
    assert bit_equal(both, oracle.bitwise_and(e, nz)) and bit_equal(both, e & nz)
    # bool bytes are exactly 0 or 1
    assert set(both.view(torch.uint8).unique().tolist()) <= {0, 1}


def test_compare_ieee_cases_and_layouts(twg):
    a = torch.tensor([0.0, -0.0, float("nan"), float("nan"), float("inf"), 1.0, -0.0, 5.0])
    b = torch.tensor([-0.0, 0.0, float("nan"), 1.0, float("inf"), float("nan"), -0.0, 5.0])
    assert bit_equal(H.binary("twg_eq_f32", a, b, out_dtype=torch.bool), torch.eq(a, b))
    for s in (0.0, -0.0, 5.0, float("nan")):
        assert bit_equal(H.unary("twg_ne_scalar_f32", a, out_dtype=torch.bool,
                                 extra=(ctypes.c_float(s),)), a.ne(s))
    g = torch.Generator().manual_seed(8)
    for n in (1, 3, 15, 16, 17, 4099):  # around the 4- and 16-element packs, misaligned
        x = torch.randint(0, 3, (n + 1,), generator=g).float()
        y = torch.randint(0, 3, (n + 1,), generator=g).float()
        assert bit_equal(H.binary("twg_eq_f32", x[1:], y[:-1], out_dtype=torch.bool),
                         torch.eq(x[1:], y[:-1]))
        m1, m2 = x > 0, y > 1
        assert bit_equal(H.binary("twg_and_u8", m1[1:], m2[:-1], out_dtype=torch.bool),
                         m1[1:] & m2[:-1])
    # broadcast and transposed compares
    X = torch.randint(0, 4, (130, 70), generator=g).float()
    row = torch.randint(0, 4, (1, 70), generator=g).float()
    assert bit_equal(H.binary("twg_eq_f32", X, row, out_dtype=torch.bool), torch.eq(X, row))
    Y = torch.randint(0, 4, (70, 130), generator=g).float()
    assert bit_equal(H.binary("twg_eq_f32", X, Y.t(), out_dtype=torch.bool), torch.eq(X, Y.t()))
    M = X > 1
    assert bit_equal(H.binary("twg_and_u8", M, (Y > 0).t(), out_dtype=torch.bool), M & (Y > 0).t())
    assert bit_equal(H.unary("twg_copy_strided", M.t(), out_dtype=torch.bool,
                             extra=(ctypes.c_int32(1),)), M.t().contiguous())


@pytest.mark.parametrize("dtype", [torch.uint8, torch.int16, torch.float32, torch.int64, torch.float64])
def test_copy_strided_every_element_size_and_layout(twg, dtype):
    # twg_copy_strided moves elements of 1, 2, 4 and 8 bytes without looking at them.  8-byte
    # elements travel as pairs of 4-byte words (one more innermost dimension) through the same
    # kernels as float32, so every layout class is checked for every size: transposed, permuted
    # with short and long innermost extents, channels-last pixels, sliced and stepped rows,
    # broadcast, sliced outputs, and an 8-dimensional view that leaves no room for the extra
    # dimension.
    g = torch.Generator().manual_seed(42 + dtype.itemsize)
    es = ctypes.c_int32(dtype.itemsize)

    def rnd(*shape):
        return (torch.randn(*shape, generator=g) * 1000).to(dtype)

    def check(view, out=None, what=""):
        _say(f"copy_strided {dtype} {what} {tuple(view.shape)} strides {view.stride()}")
        got = H.unary("twg_copy_strided", view, out=out, out_dtype=dtype, extra=(es,))
        assert torch.equal(got, view.contiguous() if out is None else view), (dtype, what)

    check(rnd(300, 200).t(), what="transposed")
    # extents and strides that are multiples of 16 elements: 1- and 2-byte elements take the tile
    # kernel with 16-byte packs on both sides (whole tiles, ragged tiles, a batch, an offset
    # that keeps the alignment and one that breaks it)
    check(rnd(320, 256).t(), what="transposed, whole packs")
    check(rnd(1088, 544).t(), what="transposed, ragged tiles")
    check(rnd(3, 160, 96).transpose(1, 2), what="batched transposes")
    check(rnd(4, 32, 48, 64).permute(0, 3, 1, 2), what="NHWC viewed as NCHW, whole packs")
    check(rnd(2, 64, 48, 32).permute(3, 1, 0, 2), what="permuted, whole packs")
    check(rnd(16 + 320 * 256)[16:].view(320, 256).t(), what="transposed, storage offset of 16")
    check(rnd(3 + 320 * 256)[3:].view(320, 256).t(), what="transposed, storage offset of 3")
    check(rnd(256, 512).t(), out=torch.zeros(512, 512, dtype=dtype)[:, :256], what="transposed into a wider output")
    # planar <-> interleaved with few channels (image batches between NCHW and NHWC): 1- and
    # 2-byte elements take strips through LDS; several strips per row with a shorter last one,
    # 2 to 32 channels, a batch, and a row length that is no whole number of packs (the gather)
    check(rnd(2, 3, 224, 224).permute(0, 2, 3, 1), what="NCHW viewed as NHWC, 3 channels")
    check(rnd(2, 224, 224, 3).permute(0, 3, 1, 2), what="NHWC viewed as NCHW, 3 channels")
    check(rnd(3, 16, 48, 48).permute(0, 2, 3, 1), what="NCHW viewed as NHWC, 16 channels")
    check(rnd(3, 48, 48, 16).permute(0, 3, 1, 2), what="NHWC viewed as NCHW, 16 channels")
    check(rnd(2, 5, 64, 80).permute(0, 2, 3, 1), what="NCHW viewed as NHWC, 5 channels")
    check(rnd(2, 64, 80, 31).permute(0, 3, 1, 2), what="NHWC viewed as NCHW, 31 channels")
    check(rnd(2, 32, 40, 40).permute(0, 2, 3, 1), what="NCHW viewed as NHWC, 32 channels")
    check(rnd(2, 1, 4096 + 272).expand(2, 7, 4096 + 272).transpose(1, 2), what="one plane for all 7 channels")
    check(rnd(2, 3, 17, 19).permute(0, 2, 3, 1), what="NCHW viewed as NHWC, ragged rows")
    # output rows that are no whole number of packs, the output dense across them (1- and 2-byte
    # elements: blocks write whole rows as one run of aligned packs with a head and a tail)
    check(rnd(3, 197, 768).transpose(1, 2), what="rows of 197")
    check(rnd(2, 33, 640).transpose(1, 2), what="rows of 33")
    check(rnd(511, 256).t(), what="rows of 511, two dimensions")
    check(rnd(5, 9, 128).transpose(1, 2), what="rows of 9")
    check(rnd(1 + 2 * 77 * 192)[1:].view(2, 77, 192).transpose(1, 2), what="rows of 77, storage offset of 1")
    check(rnd(2, 77, 192).transpose(1, 2), out=torch.zeros(1 + 2 * 192 * 77, dtype=dtype)[1:].view(2, 192, 77),
          what="rows of 77 into an output that starts off a pack")
    # the mirror image: input rows that are no whole number of packs, the input dense across them
    check(rnd(3, 768, 197).transpose(1, 2), what="input rows of 197")
    check(rnd(2, 640, 33).transpose(1, 2), what="input rows of 33")
    check(rnd(256, 511).t(), what="input rows of 511, two dimensions")
    check(rnd(5, 128, 9).transpose(1, 2), what="input rows of 9")
    check(rnd(1 + 2 * 192 * 77)[1:].view(2, 192, 77).transpose(1, 2), what="input rows of 77, storage offset of 1")
    check(rnd(2, 1000, 77).transpose(1, 2), what="input rows of 77, a last block of 40 rows")
    if dtype == torch.uint8:  # from 2^26 elements on, 1-byte elements take wider tiles
        big = torch.randint(0, 256, (8192 + 144, 8192), generator=g, dtype=torch.uint8)
        check(big.t(), what="transposed, 2^26 elements and a ragged last tile")
        del big
    check(rnd(1027, 260).t(), what="transposed, ragged")
    check(rnd(4, 30, 40, 3).permute(0, 3, 1, 2), what="NHWC viewed as NCHW")
    check(rnd(4, 3, 30, 40).permute(0, 2, 3, 1), what="NCHW viewed as NHWC")
    check(rnd(5, 33, 35, 4).permute(0, 2, 1, 3), what="pixels, h and w swapped")
    check(rnd(6, 17, 64, 70).permute(3, 1, 0, 2), what="permuted")
    check(rnd(2, 96, 56, 56).permute(0, 2, 3, 1), what="permuted, 96 channels")
    check(rnd(37, 1001)[:, 1:], what="rows from 1 on")
    check(rnd(50, 2048)[:, ::2], what="stepped rows")
    check(rnd(1, 700).expand(90, 700), what="broadcast rows")
    check(rnd(90, 1).expand(90, 700), what="one value per row")
    check(rnd(64, 128), out=torch.zeros(128, 64, dtype=dtype).t(), what="transposed output")
    check(rnd(40, 300), out=torch.zeros(40, 601, dtype=dtype)[:, 1::2], what="stepped output")
    x8 = rnd(2, 3, 2, 2, 3, 2, 2, 6)[:, ::2, :, :, ::2]
    check(x8.permute(7, 6, 5, 4, 3, 2, 1, 0), what="8 dimensions, reversed")
    check(rnd(70001)[1:], what="one dimension from 1 on")
    check(rnd((1 << 20) + 3), what="dense")


# ----------------------------------------------------------- masked_select

@pytest.mark.parametrize("p", [0.0, 0.01, 0.5, 0.99, 1.0])
@pytest.mark.parametrize("n", [1, 63, 64, 8191, 8192, 8193, (1 << 21) + 77])
def test_masked_select_bernoulli(twg, n, p):
    _say(f"masked_select n={n} p={p}")
    x = W.select_source(n, seed=4)
    m = W.bernoulli_mask(n, p, seed=n % 1000) if 0.0 < p < 1.0 else torch.full((n,), p == 1.0)
    vals, k = H.masked_select(x, m, check_guard=True)
    ref = oracle.masked_select(x, m)
    assert k == int(m.sum()) == ref.numel()
    assert bit_equal(vals, ref)
    assert bit_equal(vals, torch.masked_select(x, m))


@pytest.mark.parametrize("n,p,out_offset", [
    (1 << 25, 0.5, 0), ((1 << 25) + 3 * 131072 + 12345, 0.5, 1), ((1 << 25) + 5, 0.99, 31),
    ((1 << 25) + 8191, 0.01, 0), ((1 << 25) + 8191, 0.001, 7), ((1 << 25) + 140000, 1.0, 3),
    ((1 << 25) + 140000, 0.0, 0), ((1 << 25) + 40000, -1.0, 17), ((1 << 24) + 70000, 0.5, 0),
    ((1 << 23) + 65536 + 5, 0.5, 9), ((1 << 23) - 1, 0.99, 2), ((1 << 22) + 3, -1.0, 30),
    (1 << 21, 0.5, 1)])
def test_masked_select_large_tiles(twg, n, p, out_offset):
    # From 2^21 elements the streaming kernel runs (16384-, 65536- and, from 2^25,
    # 131072-element tiles), its last tile bounds-checked.  A shifted output pointer moves
    # every wavefront's first and last line.
    _say(f"masked_select large n={n} p={p} out_offset={out_offset}")
    x = W.select_source(n, seed=4)
    if p < 0:
        m = W.clustered_mask(n, mean_run=4096, seed=6)
    elif 0.0 < p < 1.0:
        m = W.bernoulli_mask(n, p, seed=11)
    else:
        m = torch.full((n,), p == 1.0)
    vals, k = H.masked_select(x, m, out_offset=out_offset, check_guard=True)
    assert k == int(m.sum())
    assert bit_equal(vals, torch.masked_select(x, m))


def test_masked_select_streaming_edge_patterns(twg):
    # masks that leave wavefronts, whole tiles or all but a few elements empty, and runs
    # shorter than a 128-byte line, for each streaming tile size; every output phase
    g = torch.Generator().manual_seed(12)
    for n in ((1 << 21) + 12345, (1 << 23) + 777, (1 << 25) + 131072 + 9):
        x = W.select_source(n, seed=4)
        idx = torch.arange(n)
        patterns = {
            "one in 100000": idx % 100000 == 7,
            "first only": idx == 0,
            "last only": idx == n - 1,
            "3 of 5003": idx % 5003 < 3,
            "33 of 40000": idx % 40000 < 33,
            "around tile edges": ((idx + 2) % 16384) < 4,
            "second half": idx >= n // 2,
            "one wavefront's span": (idx >= 70000) & (idx < 70000 + 2048),
            # around the density (1 in 16 per wavefront) below which a wavefront gathers
            # its elements one by one instead of streaming
            "every 16th": idx % 16 == 5,
            "every 16th and one more": (idx % 16 == 5) | (idx % 2048 == 0),
            "128 in a row per 8192": (idx % 8192 >= 384) & (idx < 512 + idx // 8192 * 8192),
            "3 percent": W.bernoulli_mask(n, 0.03, seed=21),
            "6 percent": W.bernoulli_mask(n, 0.06, seed=22),
        }
        for name, m in patterns.items():
            ref = torch.masked_select(x, m)
            for off in (0, 1, 31):
                _say(f"masked_select pattern n={n} {name} out_offset={off}")
                vals, k = H.masked_select(x, m, out_offset=off, check_guard=True)
                assert k == ref.numel() and bit_equal(vals, ref), (n, name, off)


def test_masked_select_alternating_sparse_and_dense_wavefronts(twg):
    # neighbouring 8192-element spans (one wavefront's share of a 131072-element tile) at 1% and
    # 90% selected: the gather path and the streaming loop side by side inside every tile;
    # also with spans that straddle the wavefront boundaries
    for n, span in (((1 << 25) + 131072 + 4099, 8192), ((1 << 25) + 5, 5000), ((1 << 23) + 17, 4096),
                    ((1 << 21) + 8192 + 3, 2048)):
        x = W.select_source(n, seed=4)
        m = W.alternating_density_mask(n, span=span)
        ref = torch.masked_select(x, m)
        for off in (0, 5):
            _say(f"masked_select alternating density n={n} span={span} out_offset={off}")
            vals, k = H.masked_select(x, m, out_offset=off, check_guard=True)
            assert k == ref.numel() and bit_equal(vals, ref), (n, span, off)


def test_masked_select_int64_source_that_ends_with_its_block(twg):
    # An int64 source of 2^21 + 2^18 elements fills an 18 MiB block of the allocator exactly;
    # the view x[2:] is 16-byte aligned (fast path) and its length leaves two elements in the
    # last lane's quad, whose second 16-byte half would start at the end of the block.  The
    # kernel must not fetch that half.
    n_store = (1 << 21) + (1 << 18)
    g = torch.Generator().manual_seed(77)
    x = torch.randint(-(1 << 62), 1 << 62, (n_store,), generator=g, dtype=torch.int64)
    for xv in (x[2:], x[2:-1], x[2:-3]):   # two, one and three elements in the last quad
        m = torch.rand(xv.numel(), generator=g) < 0.99
        m[-8:] = True
        _say(f"masked_select int64 view of {xv.numel()} elements at the end of its block")
        vals, k = H.masked_select(xv, m, check_guard=True)
        ref = torch.masked_select(xv, m)
        assert k == ref.numel() and bit_equal(vals, ref)
    # float64 through the same path, mask dense only at the very end
    xd = x.view(torch.float64)[2:]
    m = torch.zeros(xd.numel(), dtype=torch.bool)
    m[-3:] = True
    vals, k = H.masked_select(xd, m, check_guard=True)
    assert k == 3 and bit_equal(vals, xd[-3:])


def test_masked_select_wait_gives_up_instead_of_hanging(twg):
    # The look-back's wait is bounded.  With the ticket counter started at 1 (or 3) instead of
    # 0 the first tiles are never compacted or published, so every later tile polls a word
    # that nobody will write: it must give up after max_poll_rounds, write nothing, report -1
    # as the count and set the error word of the scratch header - and every workgroup exits.
    L = twg.load()
    g = torch.Generator().manual_seed(5)
    cases = [
        ("tile variant, 2 tiles", 16384, 0, 1),
        ("tile variant, 40 tiles", 8192 * 40 - 100, 0, 3),
        ("streaming variant, 129 tiles of 16384", (1 << 21) + 5, 0, 3),
        ("streaming variant, 257 tiles of 131072", (1 << 25) + 9, 0, 1),
        ("one element per lane (misaligned source), 3 tiles", 3 * 16384 - 7, 1, 1),
    ]
    for name, n, shift, first in cases:
        _say(f"masked_select abandoned wait: {name}")
        x = torch.rand(n + shift, generator=g)
        m = torch.rand(n, generator=g) < 0.5
        d_x, d_m = twg.to_device(x), twg.to_device(m)
        out = twg.DeviceBuffer(4 * n)
        twg.check(L.twg_fill_bytes(out.ptr, 0xAB, out.nbytes, None))
        cnt = twg.DeviceBuffer(8)
        twg.check(L.twg_fill_bytes(cnt.ptr, 0x11, 8, None))
        sb = L.twg_masked_select_scratch_bytes(n)
        scratch = twg.DeviceBuffer(sb)
        it = twg.dense_iter(n)
        twg.check(L.twg_masked_select_f32_wait_probe(out.ptr, cnt.ptr, d_x.ptr + 4 * shift, d_m.ptr,
                                                     ctypes.byref(it), scratch.ptr, sb, first, 64, None))
        twg.sync()
        assert int(cnt.download((1,), torch.int64)[0]) == -1, name
        hdr = scratch.download((2,), torch.int32)
        assert int(hdr[1]) == 1, "the error word of the scratch header is not set"
        assert bool((out.download((out.nbytes,), torch.uint8) == 0xAB).all()), "a tile that gave up wrote output"
        # the same scratch serves a normal call afterwards: every launch clears what it needs
        twg.check(L.twg_masked_select_f32(out.ptr, cnt.ptr, d_x.ptr + 4 * shift, d_m.ptr,
                                          ctypes.byref(it), scratch.ptr, sb, None))
        k = int(cnt.download((1,), torch.int64)[0])
        assert k == int(m.sum())
        assert bit_equal(out.download((k,), torch.float32), x[shift:shift + n][m])
        assert int(scratch.download((2,), torch.int32)[1]) == 0
    # the probe with nothing forced is the ordinary call
    n = 8192 * 5 + 3
    x, m = torch.rand(n, generator=g), torch.rand(n, generator=g) < 0.3
    d_x, d_m, out, cnt = twg.to_device(x), twg.to_device(m), twg.DeviceBuffer(4 * n), twg.DeviceBuffer(8)
    sb = L.twg_masked_select_scratch_bytes(n)
    scratch = twg.DeviceBuffer(sb)
    it = twg.dense_iter(n)
    twg.check(L.twg_masked_select_f32_wait_probe(out.ptr, cnt.ptr, d_x.ptr, d_m.ptr, ctypes.byref(it),
                                                 scratch.ptr, sb, 0, 0, None))
    assert int(cnt.download((1,), torch.int64)[0]) == int(m.sum())
    assert L.twg_masked_select_f32_wait_probe(out.ptr, cnt.ptr, d_x.ptr, d_m.ptr, ctypes.byref(it),
                                              scratch.ptr, sb, 256, 0, None) == twg.E_INVALID_ARG
    assert b"gave up" in L.twg_error_string(twg.E_WAIT_ABANDONED)


def test_masked_select_clustered_and_empty(twg):
    n = (1 << 22) + 1234
    x = W.select_source(n, seed=4)
    m = W.clustered_mask(n, mean_run=4096, seed=6)
    vals, k = H.masked_select(x, m)
    assert k == int(m.sum())
    assert bit_equal(vals, torch.masked_select(x, m))
    # zero elements
    vals0, k0 = H.masked_select(torch.empty(0), torch.empty(0, dtype=torch.bool))
    assert k0 == 0 and vals0.numel() == 0


def test_masked_select_misaligned_broadcast_strided(twg):
    g = torch.Generator().manual_seed(9)
    n = 50021
    x = torch.rand(n + 3, generator=g)
    m = torch.rand(n + 3, generator=g) < 0.4
    # misaligned source / mask pointers (scalar variant of the kernel)
    for xo, mo in ((1, 0), (0, 1), (3, 2)):
        vals, k = H.masked_select(x[xo:xo + n], m[mo:mo + n], check_guard=True)
        assert bit_equal(vals, torch.masked_select(x[xo:xo + n], m[mo:mo + n]))
    # reference known answers: row mask over a matrix, transposed self
    xm = torch.tensor([[0., 1., 2.], [3., 4., 5.]])
    rm = torch.tensor([True, False, True])
    assert torch.equal(H.masked_select(xm, rm, check_guard=True)[0], torch.tensor([0., 2., 3., 5.]))
    xt = torch.arange(6.).view(3, 2).t()
    assert torch.equal(H.masked_select(xt, rm, check_guard=True)[0], torch.tensor([0., 4., 1., 5.]))
    # larger broadcast / strided cases against the oracle and ATen
    x3 = torch.rand(37, 1, 50, generator=g)
    m3 = torch.rand(1, 11, 50, generator=g) < 0.5
    v, _ = H.masked_select(x3, m3)
    assert bit_equal(v, oracle.masked_select(x3, m3)) and bit_equal(v, torch.masked_select(x3, m3))
    xs = torch.rand(300, 200, generator=g).t()[::2]
    ms = (torch.rand(200, 300, generator=g) < 0.3)[::2]
    v, _ = H.masked_select(xs, ms)
    assert bit_equal(v, torch.masked_select(xs, ms))


@pytest.mark.parametrize("dtype", [torch.float32, torch.uint8, torch.int16, torch.int64])
def test_masked_select_layouts_that_are_copied_dense_first(twg, dtype):
    # From 2^16 elements on, a source or mask that is not dense in logical order (transposed,
    # sliced, broadcast along rows or columns, off its alignment) is written out dense before the
    # vectorised kernels run: same values, same order, nothing written past the k results.
    g = torch.Generator().manual_seed(77)
    rows, cols = 640, 1000
    x = (torch.randn(rows, cols, generator=g) * 1000).to(dtype)
    m = torch.rand(rows, cols, generator=g) < 0.45
    xt = (torch.randn(cols, rows, generator=g) * 1000).to(dtype).t()
    mt = (torch.rand(cols, rows, generator=g) < 0.6).t()
    wide = (torch.randn(rows, 2 * cols + 3, generator=g) * 1000).to(dtype)
    cases = [
        ("source transposed", xt, m),
        ("mask transposed", x, mt),
        ("both transposed", xt, mt),
        ("one mask row for all rows", x, m[3]),
        ("one mask value per row", x, m[:, 5:6]),
        ("one source row under a full mask", x[7], m),
        ("source stepped by 2", wide[:, 1:2 * cols:2], m),
        ("source and mask off their alignment", x.flatten()[1:-3], m.flatten()[3:-1]),
        ("three dimensions, the middle one broadcast", x.view(rows, 1, cols).expand(rows, 2, cols)[:400], m[:400].view(400, 1, cols)),
    ]
    for name, xs, ms in cases:
        _say(f"masked_select {dtype} {name}")
        vals, k = H.masked_select(xs, ms, check_guard=True)
        ref = torch.masked_select(xs, ms)
        assert k == ref.numel() and bit_equal(vals, ref), (dtype, name)
        if dtype == torch.float32:
            assert bit_equal(vals, oracle.masked_select(xs, ms)), name


def test_masked_select_rejects_small_scratch(twg):
    x = torch.rand(100000)
    m = x > 0.5
    with pytest.raises(H.capi.TwgError) as ei:
        H.masked_select(x, m, scratch_bytes=64)
    assert ei.value.code == H.capi.E_SCRATCH_SMALL


def test_invalid_iter_is_rejected(twg):
    L = twg.load()
    it = twg.dense_iter(16)
    it.numel = 17  # does not match the shape
    buf = twg.DeviceBuffer(64)
    assert L.twg_add_f32(buf.ptr, buf.ptr, buf.ptr, 1.0, ctypes.byref(it), None) == twg.E_INVALID_ARG
    it = twg.dense_iter(16)
    it.ndim = 9
    assert L.twg_add_f32(buf.ptr, buf.ptr, buf.ptr, 1.0, ctypes.byref(it), None) == twg.E_INVALID_ARG
    assert L.twg_unary_f32(99, buf.ptr, buf.ptr, ctypes.byref(twg.dense_iter(16)), None) == twg.E_INVALID_ARG


def test_entry_points_capture_into_a_hip_graph(twg):
    # A caller may record the launches on a stream of its own into a HIP graph and replay
    # them: every entry point only enqueues kernels (the scratch clear of masked_select is a
    # fill kernel, not a memset node).  Replays, with new input contents each time and eager
    # work in between, must reproduce the eager results bit for bit.
    hip = ctypes.CDLL("libamdhip64.so")
    vp = ctypes.c_void_p

    def ok(rc):
        assert rc == 0, f"HIP error {rc}"

    L = twg.load()
    stream = vp()
    ok(hip.hipStreamCreateWithFlags(ctypes.byref(stream), 1))  # hipStreamNonBlocking
    n = (1 << 21) + 4096 + 13
    g = torch.Generator().manual_seed(91)
    a_h, b_h = torch.randn(n, generator=g), torch.randn(n, generator=g)
    m_h = torch.rand(n, generator=g) < 0.37
    d_a, d_b, d_m = twg.to_device(a_h), twg.to_device(b_h), twg.to_device(m_h)
    d_sum, d_act, d_eq, d_sel = (twg.DeviceBuffer(4 * n), twg.DeviceBuffer(4 * n), twg.DeviceBuffer(n),
                                 twg.DeviceBuffer(4 * n))
    d_cnt = twg.DeviceBuffer(8)
    sb = L.twg_masked_select_scratch_bytes(n)
    d_scr = twg.DeviceBuffer(sb)
    it = twg.dense_iter(n)

    def enqueue(s):
        twg.check(L.twg_add_f32(d_sum.ptr, d_a.ptr, d_b.ptr, ctypes.c_float(1.0), ctypes.byref(it), s))
        twg.check(L.twg_unary_f32(twg.UNARY_GELU_ERF, d_act.ptr, d_sum.ptr, ctypes.byref(it), s))
        twg.check(L.twg_eq_f32(d_eq.ptr, d_a.ptr, d_b.ptr, ctypes.byref(it), s))
        twg.check(L.twg_masked_select_f32(d_sel.ptr, d_cnt.ptr, d_act.ptr, d_m.ptr, ctypes.byref(it),
                                          d_scr.ptr, sb, s))

    def results():
        k = int(d_cnt.download((1,), torch.int64)[0])
        return (d_act.download((n,), torch.float32), d_eq.download((n,), torch.uint8),
                k, d_sel.download((k,), torch.float32))

    twg.sync()
    ok(hip.hipStreamBeginCapture(stream, 1))  # hipStreamCaptureModeThreadLocal
    try:
        enqueue(stream)
    finally:
        graph = vp()
        rc_end = hip.hipStreamEndCapture(stream, ctypes.byref(graph))
    ok(rc_end)
    graph_exec = vp()
    ok(hip.hipGraphInstantiate(ctypes.byref(graph_exec), graph, None, None, ctypes.c_size_t(0)))
    try:
        for rep in range(3):
            _say(f"graph replay {rep}")
            if rep:  # new contents in the same buffers, and unrelated eager work in between
                a_h = torch.randn(n, generator=g)
                a_h[::5] = b_h[::5]
                m_h = torch.rand(n, generator=g) < (0.1 + 0.4 * rep)
                d_a.upload(a_h)
                d_m.upload(m_h)
                H.add(a_h[:1000], b_h[:1000])
            twg.sync()
            ok(hip.hipGraphLaunch(graph_exec, stream))
            ok(hip.hipStreamSynchronize(stream))
            got = results()
            for buf in (d_act, d_eq, d_sel, d_cnt):  # wipe, then the same work eagerly
                twg.check(L.twg_fill_bytes(buf.ptr, 0xCD, buf.nbytes, None))
            enqueue(None)
            twg.sync()
            want = results()
            assert got[2] == want[2] == int(m_h.sum())
            assert bit_equal(got[0], want[0]) and torch.equal(got[1], want[1]) and bit_equal(got[3], want[3])
            assert torch.equal(got[1].bool(), torch.eq(a_h, b_h))
    finally:
        hip.hipGraphExecDestroy(graph_exec)
        hip.hipGraphDestroy(graph)
        hip.hipStreamDestroy(stream)



def test_block_freed_while_a_caller_stream_still_uses_it(twg):
    # Work queued on a stream of the caller's own; the output block of its first launch is
    # recorded on that stream and freed at once, then a block of the same size is allocated and
    # overwritten on the library's stream.  The allocator must keep the freed block aside until
    # the caller's stream has passed the free (bytes_pending), so the second launch on that
    # stream still reads the sum, bit for bit.
    hip = ctypes.CDLL("libamdhip64.so")
    L = twg.load()
    stream = ctypes.c_void_p()
    assert hip.hipStreamCreateWithFlags(ctypes.byref(stream), 1) == 0  # hipStreamNonBlocking
    n = 1 << 24
    g = torch.Generator().manual_seed(17)
    a_h, b_h = torch.randn(n, generator=g), torch.randn(n, generator=g)
    d_a, d_b = twg.to_device(a_h), twg.to_device(b_h)
    d_res, d_busy = twg.DeviceBuffer(4 * n), twg.DeviceBuffer(4 * n)
    it = twg.dense_iter(n)
    twg.sync()
    base = twg.mem_stats()
    assert base["bytes_pending"] == 0
    # keep the caller's stream busy for a few milliseconds first
    for _ in range(40):
        twg.check(L.twg_add_f32(d_busy.ptr, d_a.ptr, d_b.ptr, ctypes.c_float(1.0), ctypes.byref(it), stream))
    d_sum = twg.DeviceBuffer(4 * n)
    addr = d_sum.ptr
    twg.check(L.twg_add_f32(d_sum.ptr, d_a.ptr, d_b.ptr, ctypes.c_float(1.0), ctypes.byref(it), stream))
    twg.check(L.twg_unary_f32(twg.UNARY_GELU_ERF, d_res.ptr, d_sum.ptr, ctypes.byref(it), stream))
    twg.check(L.twg_record_stream(ctypes.c_void_p(d_sum.ptr + 4096), stream))  # any address inside
    d_sum.free()
    assert twg.mem_stats()["bytes_pending"] == 4 * n
    other = twg.DeviceBuffer(4 * n)   # same size class: must not be the block still in use
    assert other.ptr != addr
    twg.check(L.twg_fill_bytes(other.ptr, 0xAB, 4 * n, None))
    assert hip.hipStreamSynchronize(stream) == 0
    twg.sync()
    # reference on the library's stream, into fresh buffers
    d_s2, d_r2 = twg.DeviceBuffer(4 * n), twg.DeviceBuffer(4 * n)
    assert twg.mem_stats()["bytes_pending"] == 0   # the caller's stream is done: reaped
    twg.check(L.twg_add_f32(d_s2.ptr, d_a.ptr, d_b.ptr, ctypes.c_float(1.0), ctypes.byref(it), None))
    twg.check(L.twg_unary_f32(twg.UNARY_GELU_ERF, d_r2.ptr, d_s2.ptr, ctypes.byref(it), None))
    got, ref = d_res.download((n,), torch.float32), d_r2.download((n,), torch.float32)
    assert bit_equal(got, ref)
    assert bool((other.download((4 * n,), torch.uint8) == 0xAB).all())
    # the library's own stream needs no record, and an unknown address is refused
    assert L.twg_record_stream(ctypes.c_void_p(d_res.ptr), None) == 0
    assert L.twg_record_stream(ctypes.c_void_p(12345), stream) == twg.E_INVALID_ARG
    assert hip.hipStreamDestroy(stream) == 0


def test_small_reads_from_several_threads(twg):
    # each reader polls a mailbox of its own: 8 threads reading different scalars and counts
    # at once must all get their own values
    import threading
    L = twg.load()
    vals = torch.arange(64, dtype=torch.int64) * 1000 + 7
    dev = twg.to_device(vals)
    n = 50000
    src = torch.arange(n, dtype=torch.float32)
    d_src = twg.to_device(src)
    errors = []

    def reader(t):
        try:
            it = twg.dense_iter(n)
            mask = (torch.arange(n) % (t + 2)) == 0
            d_mask = twg.to_device(mask)
            out = twg.DeviceBuffer(4 * n)
            sb = L.twg_masked_select_scratch_bytes(n)
            scr = twg.DeviceBuffer(sb)
            for rep in range(50):
                i = (t * 7 + rep) % 64
                got = dev.download((1,), torch.int64, byte_offset=8 * i)
                if int(got[0]) != int(vals[i]):
                    errors.append(("scalar", t, rep, int(got[0])))
                k = ctypes.c_int64(-1)
                twg.check(L.twg_masked_select_count(out.ptr, ctypes.byref(k), d_src.ptr, 4, d_mask.ptr,
                                                    ctypes.byref(it), scr.ptr, sb, None))
                if k.value != int(mask.sum()):
                    errors.append(("count", t, rep, k.value))
        except Exception as exc:  # noqa: BLE001
            errors.append(("exception", t, repr(exc)))

    threads = [threading.Thread(target=reader, args=(t,)) for t in range(8)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors[:5]
