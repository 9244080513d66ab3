"""The five benchmark configurations at their full sizes (2^28 elements), through the
C ABI.  ATen's CPU kernels are fast enough to serve as the element-by-element check
here: bit-exact for add / relu / eq / ne / bitwise_and / masked_select (ATen's CPU
kernel IS the reference's implementation of the last four, csrc/bindings.cpp:35-42,
and the correctly rounded sum for alpha = 1), tolerance checks plus size-independent
identities for gelu and silu.
"""
import ctypes

import pytest
import torch
import torch.nn.functional as F

import capi_helpers as H
import twg_workloads as W
from util import FLOOR, bit_equal, closed_form64, rel_err_ok

pytestmark = pytest.mark.gpu

N = 1 << 28


def _say(msg):
    print(msg, flush=True)


def test_full_add_contiguous(twg):
    _say("full-size add: 2^28 contiguous")
    a, b = W.add_contiguous(N, seed=0)
    got = H.add(a, b)
    assert bit_equal(got, a + b)
    # linearity spot check that does not depend on the CPU result: (a + b) - b == a
    # wherever the sum was exact, i.e. almost everywhere for same-exponent operands;
    # instead use the exact identity add(a, -a) == 0
    z = H.add(a, -a)
    assert int(torch.count_nonzero(z)) == 0


def test_full_activations(twg):
    import twg_capi as C
    _say("full-size activations: [16384, 16384] N(0, 9) with forced 0 / +-1e-30")
    x = W.activation_input(16384, 16384, seed=1)
    pick = torch.arange(0, N, 61)  # subsample for the float64 closed forms
    far = torch.nonzero(x.view(-1).abs() > 12.0).view(-1)  # and every far-tail element
    pick = torch.cat([pick, far])
    xs = x.view(-1)[pick]

    def run(op):
        return H.unary("twg_unary_f32", x, pre=(ctypes.c_int(op),))

    relu = run(C.UNARY_RELU)
    assert bit_equal(relu, torch.relu(x))
    del relu

    for name, op in (("gelu_erf", C.UNARY_GELU_ERF), ("silu", C.UNARY_SILU)):
        _say(f"  {name}")
        y = run(op)
        ok, err, bound = rel_err_ok(y.view(-1)[pick], closed_form64(name, xs), floor=FLOOR[name])
        assert ok, f"{name}: worst {float((err / bound).max())} x bound"
        ref = F.gelu(x) if name == "gelu_erf" else F.silu(x)
        assert torch.allclose(y, ref, atol=2e-6, rtol=0)
        del ref
        # identity f(x) - f(-x) == x holds for both x*Phi(x) and x*sigmoid(x)
        yn = H.unary("twg_unary_f32", -x, pre=(ctypes.c_int(op),))
        resid = (y.double() - yn.double() - x.double()).abs()
        assert bool((resid <= 4e-7 * x.abs().double() + 1e-37).all())
        # exact zeros stay zeros, the +-1e-30 entries become +-5e-31
        zeros = x == 0
        assert int(torch.count_nonzero(y[zeros])) == 0
        tiny = x.abs() == 1e-30
        assert int(tiny.sum()) > 1000
        assert bool(((y[tiny] - 0.5 * x[tiny]).abs() <= 2e-6 * 5e-31).all())
        del y, yn


def test_full_rowbias_and_transposed_add(twg):
    _say("full-size config 3: [8192, 32768] + [1, 32768], and the transposed view")
    a, bias, c = W.broadcast_add_inputs(8192, 32768, seed=2)
    assert bit_equal(H.add(a, bias), a + bias)
    at = a.as_strided((32768, 8192), (1, 32768))
    ref = at + c                       # ATen lays the result out like `at`
    assert ref.stride() == (1, 32768)
    out_like = torch.empty(8192, 32768).t()
    got = H.add(at, c, out=out_like)
    assert got.stride() == ref.stride() and bit_equal(got.contiguous(), ref.contiguous())


def test_full_mask_ops(twg):
    _say("full-size config 4: eq / ne / bitwise_and on 2^28")
    p, q, z = W.mask_inputs(N, seed=3)
    e = H.binary("twg_eq_f32", p, q, out_dtype=torch.bool)
    assert bit_equal(e, torch.eq(p, q))
    frac = e.sum().item() / N
    assert abs(frac - 1 / 16) < 1e-3
    del p, q
    nz = H.unary("twg_ne_scalar_f32", z, out_dtype=torch.bool, extra=(ctypes.c_float(0.0),))
    assert bit_equal(nz, z.ne(0.0))
    assert abs(nz.sum().item() / N - 0.7) < 1e-3
    both = H.binary("twg_and_u8", e, nz, out_dtype=torch.bool)
    assert bit_equal(both, e & nz)
    # the count of a conjunction is what masked_select would return
    assert both.sum().item() == int((e & nz).sum())


@pytest.mark.parametrize("kind", ["p0.01", "p0.5", "p0.99", "clustered"])
def test_full_masked_select(twg, kind):
    _say(f"full-size masked_select: 2^28, mask {kind}")
    x = W.select_source(N, seed=4)
    m = W.clustered_mask(N, 4096) if kind == "clustered" else W.bernoulli_mask(N, float(kind[1:]))
    vals, k = H.masked_select(x, m)
    assert k == int(m.sum())
    ref = torch.masked_select(x, m)
    assert bit_equal(vals, ref)
    # order-preservation independent of the CPU result: positions recovered from the
    # values of an index-valued source must be strictly increasing
    idx_src = torch.arange(N, dtype=torch.float32)  # exact below 2^24 only: use a window
    w = 1 << 24
    v2, k2 = H.masked_select(idx_src[:w], m[:w])
    assert k2 == int(m[:w].sum())
    assert bool((v2[1:] > v2[:-1]).all())


def test_beyond_32bit_element_indices(twg):
    # 2^31 + 4099 elements (8 GiB per fp32 operand): element indices and byte offsets no
    # longer fit 32 bits anywhere; the reference stops at u32 offsets
    # (csrc/ops/binary.h:108-124).  add, eq and masked_select against ATen bit for bit.
    n = (1 << 31) + 4099
    g = torch.Generator().manual_seed(3)
    _say("beyond 2^31: generating")
    a = torch.rand(n, generator=g)
    b = torch.rand(n, generator=g)
    _say("  add")
    got = H.add(a, b)
    assert torch.equal(got, a + b)
    del got
    _say("  eq")
    b[::3] = a[::3]
    m = torch.eq(a, b)
    assert torch.equal(H.binary("twg_eq_f32", a, b, out_dtype=torch.bool), m)
    del b
    _say("  masked_select")
    vals, k = H.masked_select(a, m)
    ref = torch.masked_select(a, m)
    assert k == ref.numel() and torch.equal(vals, ref)


# ------------------------------------------------ the same sizes through the dispatcher

def test_full_transposed_add_through_the_dispatcher(twg):
    # config 3b built on the device: the [8192, 32768] tensor viewed through as_strided with
    # transposed strides plus a contiguous [32768, 8192] tensor, added by `at + c` behind
    # device="webgpu" (at::TensorIterator picks the layout and the iteration order)
    import torch_webgpu  # noqa: F401
    _say("full-size config 3b through device=\"webgpu\"")
    a_h, bias_h, c_h = W.broadcast_add_inputs(8192, 32768, seed=2)
    a, bias, c = a_h.to("webgpu"), bias_h.to("webgpu"), c_h.to("webgpu")
    assert bit_equal((a + bias).to("cpu"), a_h + bias_h)                          # 3a
    at = torch.as_strided(a, (32768, 8192), (1, 32768))
    assert at.device.type == "webgpu" and at.stride() == (1, 32768)
    r = at + c
    ref = a_h.as_strided((32768, 8192), (1, 32768)) + c_h
    assert r.shape == ref.shape and r.stride() == ref.stride()
    assert bit_equal(r.to("cpu"), ref)
    del r
    r2 = c + at                                                                   # operands swapped
    assert bit_equal(r2.to("cpu"), ref)


@pytest.mark.parametrize("kind", ["p0.01", "p0.5", "p0.99", "clustered"])
def test_full_masked_select_through_the_dispatcher(twg, kind):
    import torch_webgpu  # noqa: F401
    _say(f"full-size masked_select through device=\"webgpu\": 2^28, mask {kind}")
    x_h = W.select_source(N, seed=4)
    m_h = W.clustered_mask(N, 4096) if kind == "clustered" else W.bernoulli_mask(N, float(kind[1:]))
    x, m = x_h.to("webgpu"), m_h.to("webgpu")
    r = torch.masked_select(x, m)
    assert r.device.type == "webgpu" and r.dim() == 1
    ref = torch.masked_select(x_h, m_h)
    assert r.numel() == ref.numel() == int(m_h.sum())
    assert bit_equal(r.to("cpu"), ref)
    # a second call right behind the first reuses the freed blocks of the pool
    r2 = torch.masked_select(x, m)
    assert bit_equal(r2.to("cpu"), ref)
