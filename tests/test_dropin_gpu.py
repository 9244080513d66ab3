"""The drop-in boundary: `import torch_webgpu`, `device="webgpu"`, the dispatcher and
the registered kernels, end to end on the GPU.

The first block restates the reference's own tests/ops suite (same inputs, same
assertions and tolerances: tests/ops/test_add.py, test_gelu.py, test_silu.py,
test_mul.py, test_reshape.py, tests/test_dev.py) including the cases the reference
keeps commented out because they crash there (empty tensors, integer dtypes).  The
rest covers what no reference test touches: bool masks, masked_select, views,
resize_, strided and broadcast add through the real at::TensorIterator.
"""
import pytest
import torch
import torch.nn.functional as F

import twg_workloads as W
from oracle import oracle
from util import FLOOR, bit_equal, closed_form64, rel_err_ok

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def backend():
    import torch_webgpu  # noqa: F401
    torch.webgpu.init()
    assert torch.webgpu.is_initialized()
    yield


def dev(t):
    return t.to(device="webgpu")


# ------------------------------------------------- the reference's tests/ops suite

def test_add_happy_path():  # tests/ops/test_add.py:5-10
    a = torch.tensor([-1.5, 2.7, 1.0, 2.0], device="webgpu")
    b = torch.tensor([-1.0, 0.9, 1.1, -2.1], device="webgpu")
    result = a + b
    assert result.device.type == "webgpu"
    expected = torch.tensor([-2.5, 3.6, 2.1, -0.1], device="cpu")
    assert torch.allclose(result.to("cpu"), expected)


GELU_SILU_INPUTS = [[-1.0, 0.0, 1.0, 2.0], [[0.5, -0.5], [1.5, -1.5]], [2.0], [0.0]]


@pytest.mark.parametrize("data", GELU_SILU_INPUTS)
def test_gelu_reference_cases(data):  # tests/ops/test_gelu.py:6-53, atol 1e-3
    a = torch.tensor(data, dtype=torch.float32)
    result = F.gelu(dev(a)).to("cpu")
    assert torch.allclose(result, F.gelu(a), atol=1e-3)
    assert torch.allclose(result, F.gelu(a), atol=1e-6)  # the erf kernel is far inside it
    tanh = F.gelu(dev(a), approximate="tanh").to("cpu")  # the reference's actual formula
    assert torch.allclose(tanh, F.gelu(a), atol=1e-3)
    assert torch.allclose(tanh, F.gelu(a, approximate="tanh"), atol=1e-6)


@pytest.mark.parametrize("data", GELU_SILU_INPUTS)
def test_silu_reference_cases(data):  # tests/ops/test_silu.py:5-52, atol 1e-6
    a = torch.tensor(data, dtype=torch.float32)
    result = F.silu(dev(a)).to("cpu")
    assert torch.allclose(result, F.silu(a), atol=1e-6)


@pytest.mark.parametrize("fn", [F.gelu, F.silu, torch.relu])
def test_activation_empty_and_int_dtype(fn):
    # commented out in the reference because they segfault / are not rejected there
    # (tests/ops/test_gelu.py:56-71, test_silu.py:55-71)
    e = fn(dev(torch.tensor([], dtype=torch.float32))).to("cpu")
    assert e.numel() == 0
    with pytest.raises(RuntimeError):
        fn(dev(torch.tensor([1, 2, 3], dtype=torch.int32)))


def test_mul_reference_cases():  # tests/ops/test_mul.py:6-70
    a = dev(torch.tensor([1, 2, 3], dtype=torch.float32))
    b = dev(torch.tensor([4, 5, 6], dtype=torch.float32))
    expected = torch.tensor([4, 10, 18], dtype=torch.float32)
    assert torch.all(torch.mul(a, b).to("cpu") == expected)
    assert torch.all((a * b).to("cpu") == expected)
    m = dev(torch.tensor([[1, 2], [3, 4]], dtype=torch.float32))
    v = dev(torch.tensor([10, 20], dtype=torch.float32))
    assert torch.all(torch.mul(m, v).to("cpu") == torch.tensor([[10., 40.], [30., 80.]]))
    s = dev(torch.tensor([1, -2, 3], dtype=torch.float32))
    assert torch.all(torch.mul(s, 2).to("cpu") == torch.tensor([2., -4., 6.]))
    z = dev(torch.tensor([0, 1, 2], dtype=torch.float32))
    assert torch.all(torch.mul(z, dev(torch.zeros(3))).to("cpu") == torch.zeros(3))
    with pytest.raises(RuntimeError):
        torch.mul(a, m)  # shapes (3,) and (2, 2) do not broadcast
    empty = torch.mul(dev(torch.tensor([])), dev(torch.tensor([]))).to("cpu")  # test_mul.py:73-84
    assert empty.numel() == 0


def test_reshape_reference_cases():  # tests/ops/test_reshape.py:6-44
    a = dev(torch.arange(6, dtype=torch.float32))
    assert torch.all(torch.reshape(a, (2, 3)).to("cpu") == torch.tensor([[0., 1., 2.], [3., 4., 5.]]))
    b = dev(torch.arange(8, dtype=torch.float32))
    assert torch.all(torch.reshape(b, (2, -1)).to("cpu") ==
                     torch.tensor([[0., 1., 2., 3.], [4., 5., 6., 7.]]))
    c = dev(torch.tensor([[1, 2], [3, 4]], dtype=torch.float32))
    assert torch.all(torch.reshape(c, (-1,)).to("cpu") == torch.tensor([1., 2., 3., 4.]))
    with pytest.raises(RuntimeError):
        torch.reshape(a, (4, 2))
    with pytest.raises(RuntimeError):
        torch.reshape(a, (0, 6))
    # a reshape that cannot alias goes through clone -> strided device copy
    t = torch.arange(12, dtype=torch.float32).view(3, 4)
    assert torch.equal(torch.reshape(dev(t).t(), (12,)).to("cpu"), t.t().reshape(12))
    assert torch.equal(dev(t).view(4, 3).to("cpu"), t.view(4, 3))


def test_add_then_relu_vector():  # tests/test_dev.py:8-18 without the compile backend
    a = torch.tensor([-1.5, 2.7, 1.0, 2.0], device="webgpu")
    b = torch.tensor([-1.0, 0.9, 1.1, -2.1], device="webgpu")
    expected = torch.tensor([0, 3.6, 2.1, 0])
    assert torch.allclose(torch.relu(a + b).to("cpu"), expected)
    assert torch.allclose(torch.ops.webgpu.fused_add_relu(a, b).to("cpu"), expected)
    buf = torch.ops.webgpu.create_buffer([4], [1], torch.float32)
    assert buf.device.type == "webgpu" and buf.shape == (4,)
    torch.ops.webgpu.write_buffer(buf, torch.tensor([1., 2., 3., 4.]))
    assert torch.equal(buf.to("cpu"), torch.tensor([1., 2., 3., 4.]))


# ------------------------------------------------------------- copies and storage

def test_copy_round_trips():
    g = torch.Generator().manual_seed(21)
    for t in (torch.randn(1 << 20, generator=g), torch.rand(100003, generator=g) < 0.5,
              torch.randint(0, 255, (777,), generator=g, dtype=torch.uint8),
              torch.randint(-5, 5, (31, 7), generator=g), torch.randn(3, 5, 7, generator=g).double()):
        d = dev(t)
        assert d.device.type == "webgpu" and d.dtype == t.dtype and d.shape == t.shape
        assert bit_equal(d.to("cpu"), t)
        assert bit_equal(d.cpu(), t)
    # non-contiguous host source, non-contiguous host destination, storage offsets
    src = torch.randn(64, 48, generator=g)
    assert bit_equal(dev(src.t()).to("cpu"), src.t().contiguous())
    assert bit_equal(dev(src[3:40:2, 5:])[1:].to("cpu"), src[3:40:2, 5:][1:].contiguous())
    host = torch.zeros(48, 64).t()
    host.copy_(dev(src))
    assert bit_equal(host.contiguous(), src)
    d = dev(src)
    d[2:5].copy_(torch.ones(3, 48))           # host -> offset view of a device tensor
    src[2:5] = 1.0
    assert bit_equal(d.to("cpu"), src)
    d2 = torch.empty_like(d)
    d2.copy_(d)                               # device -> device, dense
    d2.t()[:, :8].copy_(d.t()[:, 8:16])       # device -> device, strided
    src2 = src.clone()
    src2.t()[:, :8] = src.t()[:, 8:16]
    assert bit_equal(d2.to("cpu"), src2)
    assert bit_equal(d.to("cpu", dtype=torch.float64), src.double())  # cast on the way down
    assert bit_equal(dev(src.double()).to(torch.float64).cpu(), src.double())
    assert bit_equal(dev(src).clone().contiguous().cpu(), src)
    # broadcasting copy_
    row = dev(torch.arange(48, dtype=torch.float32))
    d.copy_(row)
    assert bit_equal(d.to("cpu"), torch.arange(48.).expand(64, 48).contiguous())


def test_empty_strided_resize_as_strided():
    e = torch.empty(3, 5, device="webgpu")
    assert e.shape == (3, 5) and e.is_contiguous() and e.dtype == torch.float32
    es = torch.empty_strided((3, 5), (1, 3), device="webgpu", dtype=torch.bool)
    assert es.stride() == (1, 3) and es.dtype == torch.bool
    z = torch.empty(0, device="webgpu")
    assert z.numel() == 0 and z.to("cpu").numel() == 0
    # resize_: growth keeps the old contents, shrinking keeps the storage
    t = dev(torch.arange(6, dtype=torch.float32))
    ptr = t.data_ptr()
    t.resize_(4)
    assert t.data_ptr() == ptr and torch.equal(t.to("cpu"), torch.arange(4.))
    t.resize_(2, 3)
    assert torch.equal(t.to("cpu"), torch.arange(6.).view(2, 3))
    t.resize_(100000)
    assert torch.equal(t[:6].to("cpu"), torch.arange(6.))
    # as_strided: same metadata as on the CPU, shared storage, bounds enforced
    base = torch.arange(24, dtype=torch.float32)
    d = dev(base)
    for size, stride, off in (((4, 6), (1, 4), 0), ((3, 2), (6, 1), 5), ((2, 2, 2), (8, 2, 1), 3),
                              ((5,), (0,), 7), ((0, 3), (3, 1), 24)):
        v = torch.as_strided(d, size, stride, off)
        c = torch.as_strided(base, size, stride, off)
        assert v.shape == c.shape and v.stride() == c.stride() and v.storage_offset() == off
        assert v.untyped_storage().data_ptr() == d.untyped_storage().data_ptr()
        assert bit_equal(v.to("cpu"), c.contiguous())
    for size, stride, off in (((4, 6), (1, 4), 2), ((25,), (1,), 0), ((2,), (1,), 24), ((3,), (-1,), 1)):
        assert not oracle.as_strided_fits(size, stride, off, 24)
        with pytest.raises(RuntimeError):
            torch.as_strided(d, size, stride, off)
    assert oracle.as_strided_fits((3,), (-1,), 2, 24)  # negative strides are admitted when they fit


def test_scalar_readback_and_printing():
    t = dev(torch.tensor([0.0, 1.5, -2.0, 0.0]))
    assert t[1].item() == 1.5 and float(t[2]) == -2.0
    assert t.tolist() == [0.0, 1.5, -2.0, 0.0]
    assert (t + t)[1].item() == 3.0
    with pytest.raises((RuntimeError, ValueError)):
        t.item()
    text = repr(t)
    assert "1.5" in text and "device='webgpu:0'" in text
    assert "True" in repr(t.ne(0.0))
    assert str(torch.empty(0, device="webgpu")).startswith("tensor([]")


def test_allocator_reuses_blocks():
    a = dev(torch.randn(1 << 18))
    torch.webgpu.synchronize()
    before = torch.webgpu.memory_stats()
    for _ in range(10):
        b = a + a
        del b
    after = torch.webgpu.memory_stats()
    assert after["n_device_mallocs"] - before["n_device_mallocs"] <= 1
    assert after["n_cache_hits"] - before["n_cache_hits"] >= 9
    torch.webgpu.empty_cache()
    assert torch.webgpu.memory_stats()["bytes_cached"] == 0
    assert torch.equal((a + a).to("cpu"), a.to("cpu") * 2)


# ------------------------------------------------------------------ add variants

def test_add_forms_match_oracle():
    a_h, b_h = W.add_contiguous(1 << 20, seed=0)  # config 1, incl. the copy_ round trip
    a, b = dev(a_h), dev(b_h)
    assert bit_equal((a + b).to("cpu"), oracle.add(a_h, b_h))
    assert bit_equal(torch.add(a, b, alpha=2.5).to("cpu"), oracle.add(a_h, b_h, alpha=2.5))
    out = torch.empty(0, device="webgpu")
    torch.add(a, b, out=out)  # resized by the iterator
    assert bit_equal(out.to("cpu"), a_h + b_h)
    c = a.clone()
    c.add_(b)
    assert bit_equal(c.to("cpu"), a_h + b_h)
    c += b
    assert bit_equal(c.to("cpu"), (a_h + b_h) + b_h)
    assert bit_equal((a + 1.5).to("cpu"), a_h + 1.5)
    assert bit_equal((1.5 + a).to("cpu"), 1.5 + a_h)
    assert bit_equal(torch.add(a, 3.0, alpha=0.5).to("cpu"), oracle.add(a_h, torch.full_like(a_h, 3.0), alpha=0.5))
    assert bit_equal(torch.add(torch.tensor(2.0), a, alpha=3.0).to("cpu"),
                     oracle.add(torch.full_like(a_h, 2.0), a_h, alpha=3.0))
    assert bit_equal((a * 0.5).to("cpu"), a_h * 0.5)
    with pytest.raises(RuntimeError):
        dev(torch.ones(3)) + dev(torch.ones(4))
    with pytest.raises(RuntimeError):
        dev(torch.ones(3, dtype=torch.int64)) + dev(torch.ones(3, dtype=torch.int64))


def test_add_broadcast_and_transposed_config3():
    rows, cols = 256, 1024
    a_h, bias_h, c_h = W.broadcast_add_inputs(rows, cols, seed=2)
    a, bias, c = dev(a_h), dev(bias_h), dev(c_h)
    assert bit_equal((a + bias).to("cpu"), oracle.add(a_h, bias_h))                # 3a
    at_h = a_h.as_strided((cols, rows), (1, cols))
    at = a.as_strided((cols, rows), (1, cols))
    r = at + c                                                                     # 3b
    assert r.shape == (cols, rows)
    assert bit_equal(r.to("cpu"), oracle.add(at_h, c_h))
    assert bit_equal((c + at).to("cpu"), oracle.add(c_h, at_h))
    col = dev(a_h[:, :1].contiguous())
    assert bit_equal((a + col).to("cpu"), a_h + a_h[:, :1])
    assert bit_equal((a[::2, 3:700:3] + bias[:, 3:700:3]).to("cpu"), a_h[::2, 3:700:3] + bias_h[:, 3:700:3])
    x5 = torch.randn(3, 1, 5, 1, 7)
    y5 = torch.randn(1, 4, 1, 6, 7)
    assert bit_equal((dev(x5) + dev(y5)).to("cpu"), x5 + y5)


# ------------------------------------------------------------ activations, masks

@pytest.mark.parametrize("name", ["gelu_erf", "gelu_tanh", "silu", "relu"])
def test_activations_config2_reduced(name):
    x_h = W.activation_input(512, 2048, seed=1)
    x = dev(x_h)
    if name == "relu":
        assert bit_equal(torch.relu(x).to("cpu"), oracle.relu(x_h))
        y = x.clone()
        y.relu_()
        assert bit_equal(y.to("cpu"), torch.relu(x_h))
        return
    fn = {"gelu_erf": lambda t: F.gelu(t), "gelu_tanh": lambda t: F.gelu(t, approximate="tanh"),
          "silu": F.silu}[name]
    got = fn(x).to("cpu")
    ok, err, bound = rel_err_ok(got, closed_form64(name, x_h), floor=FLOOR[name])
    assert ok
    # non-contiguous input keeps its layout (empty_like) and its values
    got_t = fn(x.t()).to("cpu")
    assert got_t.shape == (2048, 512) and bit_equal(got_t, got.t().contiguous())
    out = torch.empty(0, device="webgpu")
    if name == "silu":
        torch.ops.aten.silu.out(x, out=out)
    else:
        torch.ops.aten.gelu.out(x, approximate="none" if name == "gelu_erf" else "tanh", out=out)
    assert bit_equal(out.to("cpu"), got)
    with pytest.raises(RuntimeError):
        F.gelu(x, approximate="bogus")


def test_mask_ops_config4_reduced():
    p_h, q_h, z_h = W.mask_inputs((1 << 20) + 3, seed=3)
    p, q, z = dev(p_h), dev(q_h), dev(z_h)
    e = torch.eq(p, q)
    assert e.dtype == torch.bool and e.device.type == "webgpu"
    assert bit_equal(e.to("cpu"), oracle.eq(p_h, q_h))
    assert bit_equal((p == q).to("cpu"), torch.eq(p_h, q_h))
    nz = z.ne(0.0)
    assert bit_equal(nz.to("cpu"), oracle.ne_scalar(z_h, 0.0))
    assert bit_equal((z != 0).to("cpu"), z_h != 0)
    both = e & nz
    assert both.dtype == torch.bool and bit_equal(both.to("cpu"), oracle.bitwise_and(e.to("cpu"), nz.to("cpu")))
    assert bit_equal(torch.bitwise_and(e, nz).to("cpu"), torch.eq(p_h, q_h) & (z_h != 0))
    out = torch.empty(0, dtype=torch.bool, device="webgpu")
    torch.eq(p, q, out=out)
    assert bit_equal(out.to("cpu"), torch.eq(p_h, q_h))
    # IEEE corner cases
    a = torch.tensor([0.0, -0.0, float("nan"), float("nan"), float("inf"), 1.0])
    b = torch.tensor([-0.0, 0.0, float("nan"), 1.0, float("inf"), float("nan")])
    assert bit_equal(torch.eq(dev(a), dev(b)).to("cpu"), torch.eq(a, b))
    assert bit_equal(dev(a).ne(0.0).to("cpu"), a.ne(0.0))
    assert bit_equal(torch.eq(dev(a).view(6, 1), dev(b).view(1, 6)).to("cpu"), torch.eq(a.view(6, 1), b.view(1, 6)))
    assert bit_equal(dev(a).abs().to("cpu"), a.abs())
    i = torch.tensor([1, 2, 1 << 40], dtype=torch.int64)
    assert bit_equal(torch.eq(dev(i), dev(i.flip(0))).to("cpu"), torch.eq(i, i.flip(0)))


@pytest.mark.parametrize("p", [0.0, 0.01, 0.5, 0.99, 1.0])
def test_masked_select_config5_reduced(p):
    n = (1 << 21) + 17
    x_h = W.select_source(n, seed=4)
    m_h = W.bernoulli_mask(n, p) if 0 < p < 1 else torch.full((n,), p == 1.0)
    x, m = dev(x_h), dev(m_h)
    r = torch.masked_select(x, m)
    assert r.device.type == "webgpu" and r.dim() == 1 and r.dtype == torch.float32
    assert r.shape[0] == int(m_h.sum())
    assert bit_equal(r.to("cpu"), oracle.masked_select(x_h, m_h))
    assert bit_equal(r.to("cpu"), torch.masked_select(x_h, m_h))


def test_masked_select_semantics():
    x_h = torch.tensor([[0., 1., 2.], [3., 4., 5.]])
    m_h = torch.tensor([True, False, True])
    x, m = dev(x_h), dev(m_h)
    assert torch.equal(torch.masked_select(x, m).to("cpu"), torch.tensor([0., 2., 3., 5.]))
    xt = dev(torch.arange(6.).view(3, 2)).t()  # transposed self: logical row-major order
    assert torch.equal(torch.masked_select(xt, m).to("cpu"), torch.tensor([0., 4., 1., 5.]))
    assert torch.masked_select(x, dev(torch.zeros(2, 3, dtype=torch.bool))).shape == (0,)
    with pytest.raises(RuntimeError, match="expected BoolTensor for mask"):
        torch.masked_select(x, dev(torch.ones(2, 3)))
    cl = W.clustered_mask(300000, mean_run=512, seed=6)
    src = W.select_source(300000, seed=7)
    assert bit_equal(torch.masked_select(dev(src), dev(cl)).to("cpu"), torch.masked_select(src, cl))
    out = torch.empty(0, device="webgpu")
    torch.masked_select(dev(src), dev(cl), out=out)
    assert bit_equal(out.to("cpu"), torch.masked_select(src, cl))
    # what tensor printing does (torch/_tensor_str.py): select the finite non-zero entries
    t = dev(torch.tensor([0.0, 1.5, -2.0, 0.0]))
    assert torch.equal(torch.masked_select(t, t.ne(0)).to("cpu"), torch.tensor([1.5, -2.0]))
    assert torch.equal(torch.masked_select(t, torch.eq(t, t) & t.ne(0)).to("cpu"),
                       torch.tensor([1.5, -2.0]))
    # int32 sources are moved bit for bit by the same kernel (patterns that would be NaNs
    # or subnormals as floats included), and so are 1-, 2- and 8-byte elements
    ints = torch.randint(-2 ** 31, 2 ** 31 - 1, (70001,), dtype=torch.int64).to(torch.int32)
    ints[:4] = torch.tensor([0x7FC00001, -0x00800000, 1, -1], dtype=torch.int32)
    im = W.bernoulli_mask(70001, 0.3, seed=9)
    got = torch.masked_select(dev(ints), dev(im))
    assert got.dtype == torch.int32 and torch.equal(got.cpu(), torch.masked_select(ints, im))
    got = torch.masked_select(dev(ints.long()), dev(im))
    assert got.dtype == torch.int64 and torch.equal(got.cpu(), torch.masked_select(ints.long(), im))
    with pytest.raises(RuntimeError, match="16 bytes"):
        torch.masked_select(dev(ints.to(torch.complex128)), dev(im))


def test_random_views_through_the_dispatcher():
    # Seeded random layouts built ON the device with the same view calls as on the CPU
    # (permute, stepped slices, expand): as_strided, at::TensorIterator's reordering and
    # merging, and every kernel family behind add / eq / masked_select must agree with ATen.
    import random
    rng = random.Random(4321)
    g = torch.Generator().manual_seed(99)
    extents = (1, 2, 3, 4, 5, 8, 16, 63, 64, 65, 128, 260)

    def make(shape):
        nd = len(shape)
        perm = rng.sample(range(nd), nd)
        steps = [rng.choice((1, 1, 1, 2, 3)) for _ in range(nd)]
        phys = [shape[perm[i]] * steps[perm[i]] for i in range(nd)]
        base = torch.randint(-8, 8, phys, generator=g).float()
        inv = [perm.index(d) for d in range(nd)]
        index = tuple(slice(None, None, steps[d]) for d in range(nd))
        return base.permute(*inv)[index], dev(base).permute(*inv)[index]

    for case in range(60):
        nd = rng.randint(1, 5)
        shape = [rng.choice(extents) for _ in range(nd)]
        while torch.Size(shape).numel() > (1 << 17):
            shape[rng.randrange(nd)] = rng.choice(extents[:6])
        bshape = [1 if rng.random() < 0.3 else e for e in shape]
        (a, da), (b, db) = make(shape), make(bshape)
        print(f"views {case}: a {tuple(a.shape)}/{a.stride()} b {tuple(b.shape)}/{b.stride()}", flush=True)
        assert da.stride() == a.stride() and db.stride() == b.stride()
        assert bit_equal((da + db).cpu(), a + b)
        assert bit_equal(torch.add(da, db, alpha=-2.0).cpu(), torch.add(a, b, alpha=-2.0))
        assert torch.equal(torch.eq(da, db).cpu(), torch.eq(a, b))
        assert bit_equal(torch.relu(da).cpu(), torch.relu(a))
        if case % 3 == 0:
            m, dm = torch.eq(a, b), torch.eq(da, db)
            assert bit_equal(torch.masked_select(da, dm).cpu(), torch.masked_select(a, m))
            assert bit_equal(torch.masked_select(db, dm).cpu(), torch.masked_select(b, m))


def test_dtype_conversions_stay_on_the_device():
    # t.to(dtype) / t.float() / mask.long() on webgpu tensors, and copy_ between host and
    # device tensors of different dtypes: all ten dtypes both ways, against ATen's CPU result.
    # Pairs without a direct kernel are composed of two (through int64 or float32).
    g = torch.Generator().manual_seed(31)
    dtypes = (torch.bool, torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64,
              torch.float16, torch.bfloat16, torch.float32, torch.float64)
    n = 5003
    for src_t in dtypes:
        if src_t == torch.bool:
            a = torch.rand(n, generator=g) < 0.5
        elif src_t.is_floating_point:
            a = (torch.rand(n, generator=g, dtype=torch.float64) * 100).to(src_t)
            a[:6] = torch.tensor([0.0, -0.0, 0.5, 0.999, 2.5, 99.5]).to(src_t)
        else:
            a = torch.randint(0, 101, (n,), generator=g).to(src_t)
        da = dev(a)
        assert da.dtype == src_t
        for dst_t in dtypes:
            ref = a.to(dst_t)
            got = da.to(dst_t)
            assert got.device.type == "webgpu" and got.dtype == dst_t
            assert bit_equal(got.cpu(), ref), (src_t, dst_t)
            # host -> device and device -> host with conversion on the way
            up = torch.empty(n, dtype=dst_t, device="webgpu").copy_(a)
            assert bit_equal(up.cpu(), ref), ("h2d", src_t, dst_t)
            down = torch.empty(n, dtype=dst_t).copy_(da)
            assert bit_equal(down, ref), ("d2h", src_t, dst_t)
    # float64 -> bool keeps values that vanish in float32; strided views convert too
    d = dev(torch.tensor([1e-300, 0.0, -0.0, 5e-324], dtype=torch.float64))
    assert d.to(torch.bool).cpu().tolist() == [True, False, False, True]
    m = torch.rand(64, 48, generator=g) < 0.3
    assert bit_equal(dev(m).t().float().cpu(), m.t().float())
    assert bit_equal(dev(m)[::2, 1::3].long().cpu(), m[::2, 1::3].long())
    # the path's own ops accept the converted tensors
    x = torch.randn(1000, generator=g, dtype=torch.float64)
    assert bit_equal((dev(x).float() + dev(x).float()).cpu(), x.float() + x.float())


def test_reshape_of_strided_int64_upload():  # tests/test_reshape.py:6-14
    storage = torch.arange(200, device="cpu")
    a_cpu = torch.as_strided(storage, size=(2, 3, 4), stride=(20, 6, 1))
    a = a_cpu.to("webgpu")
    with torch.no_grad():
        b = a.reshape((4, 6))
    assert b.shape == (4, 6) and b.dtype == torch.int64 and b.device.type == "webgpu"
    assert torch.equal(b.to("cpu"), a_cpu.reshape((4, 6)))


def test_mask_ops_take_every_dtype():
    # the reference sends eq / ne / bitwise_and / masked_select to ATen's CPU kernels
    # (csrc/bindings.cpp:36-42), which accept any dtype and promote mixed operands
    g = torch.Generator().manual_seed(9)
    ints = (torch.bool, torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64)
    floats = (torch.float16, torch.bfloat16, torch.float32, torch.float64)
    n = 3001
    for dt in ints + floats:
        a = torch.randint(0, 4, (n,), generator=g).to(dt)
        b = torch.randint(0, 4, (n,), generator=g).to(dt)
        wa, wb = a.to("webgpu"), b.to("webgpu")
        assert torch.equal(torch.eq(wa, wb).to("cpu"), torch.eq(a, b)), dt
        assert torch.equal(wa.ne(1).to("cpu"), a.ne(1)), dt
        assert torch.equal(wa.ne(0.5).to("cpu"), a.ne(0.5)), dt
        m = torch.rand(n, generator=g) < 0.5
        got = torch.masked_select(wa, m.to("webgpu"))
        assert got.dtype == dt and torch.equal(got.to("cpu"), torch.masked_select(a, m)), dt
        if dt != torch.bool:
            neg = (a.to(torch.float64) - 2).to(dt) if dt != torch.uint8 else a
            got = neg.to("webgpu").abs()
            assert got.dtype == dt and torch.equal(got.to("cpu"), neg.abs()), dt
        if dt in ints:
            got = torch.bitwise_and(wa, wb)
            assert got.dtype == dt and torch.equal(got.to("cpu"), torch.bitwise_and(a, b)), dt
    # mixed dtypes follow ATen's promotion
    i32 = torch.tensor([1, 2, 3, 16777217], dtype=torch.int32)
    f32 = torch.tensor([1.0, 2.5, 3.0, 16777216.0])
    assert torch.equal(torch.eq(i32.to("webgpu"), f32.to("webgpu")).to("cpu"), torch.eq(i32, f32))
    u8 = torch.tensor([1, 2, 255, 7], dtype=torch.uint8)
    got = torch.bitwise_and(u8.to("webgpu"), i32.to("webgpu"))
    assert got.dtype == torch.int32 and torch.equal(got.to("cpu"), torch.bitwise_and(u8, i32))
    bm = torch.tensor([True, False, True, True])
    got = torch.bitwise_and(bm.to("webgpu"), u8.to("webgpu"))
    assert got.dtype == torch.uint8 and torch.equal(got.to("cpu"), torch.bitwise_and(bm, u8))
    assert torch.equal(bm.to("webgpu").ne(1).to("cpu"), bm.ne(1))
    with pytest.raises(RuntimeError):
        torch.bitwise_and(f32.to("webgpu"), f32.to("webgpu"))
    # the scalar is converted like a C cast: wrapped around for integers
    w = torch.tensor([44, 1], dtype=torch.uint8)
    assert torch.equal(w.to("webgpu").ne(300).to("cpu"), w.ne(300))
    w = torch.tensor([-1, 1], dtype=torch.int8)
    assert torch.equal(w.to("webgpu").ne(255).to("cpu"), w.ne(255))
    assert torch.equal(bm.to("webgpu").ne(2).to("cpu"), bm.ne(2))
    big = torch.tensor([16777217], dtype=torch.int32)
    assert torch.equal(big.to("webgpu").ne(16777216.0).to("cpu"), big.ne(16777216.0))


def test_masked_select_lays_out_large_strided_operands_densely():
    # from 2^16 elements on, broadcast masks and strided sources are made dense on the device
    # before the compaction; order and values must be those of the logical row-major walk.
    # The views are built on the device with the same calls as on the CPU.
    g = torch.Generator().manual_seed(12)
    R, C = 512, 256
    x = torch.randn(R, C, generator=g)
    wide = torch.randn(R, 2 * C, generator=g)
    m_rc = torch.rand(R, C, generator=g) < 0.5
    m_cr = torch.rand(C, R, generator=g) < 0.3
    m_c = torch.rand(C, generator=g) < 0.5
    m_r1 = torch.rand(R, 1, generator=g) < 0.5
    cases = (
        (x, lambda t: t, m_c, lambda t: t),
        (x, lambda t: t, m_r1, lambda t: t),
        (x, lambda t: t.t(), m_cr, lambda t: t),
        (wide, lambda t: t[:, :C], m_rc, lambda t: t),
        (wide, lambda t: t[:, 1::2], m_cr, lambda t: t.t()),
        (x, lambda t: t[:1], m_rc, lambda t: t),            # source broadcast over the mask
    )
    for src, sv, m, mv in cases:
        want = torch.masked_select(sv(src), mv(m))
        d_src, d_m = sv(dev(src)), mv(dev(m))
        assert d_src.stride() == sv(src).stride() and d_m.stride() == mv(m).stride()
        got = torch.masked_select(d_src, d_m)
        assert bit_equal(got.to("cpu"), want), (d_src.shape, d_src.stride(), d_m.stride())


# ------------------------------------------------------------ overlap and out= checks

def test_shifted_self_copy_raises_instead_of_corrupting():
    # two dense views of one storage, one element apart: ATen raises a partial-overlap
    # error for this copy on the CPU, and the device path must not memcpy over itself
    x_h = torch.arange(1000, dtype=torch.float32)
    with pytest.raises(RuntimeError, match="single memory location|overlap"):
        y = x_h.clone()
        y[1:].copy_(y[:-1])
    x = dev(x_h)
    with pytest.raises(RuntimeError, match="single memory location|overlap"):
        x[1:].copy_(x[:-1])
    assert bit_equal(x.to("cpu"), x_h)           # nothing was written
    x[:].copy_(x)                                # the same range onto itself is a no-op
    assert bit_equal(x.to("cpu"), x_h)
    a, b = x[:500], x[500:]                      # disjoint halves still copy
    a.copy_(b)
    assert bit_equal(x.to("cpu")[:500], x_h[500:])


def test_masked_select_out_is_validated():
    src_h = W.select_source(5000, seed=7)
    m_h = W.bernoulli_mask(5000, 0.3)
    src, m = dev(src_h), dev(m_h)
    with pytest.raises(RuntimeError, match="same scalar type"):
        torch.masked_select(src, m, out=torch.empty(0, dtype=torch.float64, device="webgpu"))
    with pytest.raises(RuntimeError):
        torch.masked_select(src, m, out=torch.empty(0))          # a CPU tensor as out
    with pytest.raises(RuntimeError, match="single memory location|overlap"):
        torch.masked_select(src, m, out=src)
    out = torch.empty(3, device="webgpu")
    torch.masked_select(src, m, out=out)
    assert bit_equal(out.to("cpu"), torch.masked_select(src_h, m_h))
    # an out= with room for every element receives the values in place (no temporary, no copy)
    big = torch.empty(6000, device="webgpu")
    where = big.data_ptr()
    torch.masked_select(src, m, out=big)
    assert big.data_ptr() == where and big.shape == (int(m_h.sum()),)
    assert bit_equal(big.to("cpu"), torch.masked_select(src_h, m_h))
    none = torch.empty(10, device="webgpu")
    torch.masked_select(src, dev(torch.zeros(5000, dtype=torch.bool)), out=none)
    assert none.shape == (0,)
