"""Pins the CPU oracle (oracle/twg_oracle.c) before anything is compared against it.

Sources of truth, none of which is the oracle's own formula retyped:
  * the reference's known-answer vectors (tests/ops/test_add.py:6-9,
    test_mul.py:6-63, test_gelu.py, test_silu.py, tests/test_dev.py:8-18);
  * ATen's CPU kernels, which are the reference's implementation of eq / ne /
    bitwise_and / masked_select (csrc/bindings.cpp:35-42) and give IEEE-exact add;
  * closed forms at 50 digits (tests/golden/activations_mp.json);
  * brute force over small shapes for the index walk.
Runs on the CPU only.
"""
import itertools

import pytest
import torch
import torch.nn.functional as F

from oracle import oracle
from util import bit_equal, load_activation_golden, rel_err_ok, ulp_diff


def test_add_reference_vector():
    # tests/ops/test_add.py:6-9 and README.md:20-24
    a = torch.tensor([-1.5, 2.7, 1.0, 2.0])
    b = torch.tensor([-1.0, 0.9, 1.1, -2.1])
    expected = torch.tensor([-2.5, 3.6, 2.1, -0.1])
    assert torch.allclose(oracle.add(a, b), expected)


def test_mul_reference_vectors():
    # tests/ops/test_mul.py:6-63
    assert torch.equal(oracle.mul(torch.tensor([1., 2., 3.]), torch.tensor([4., 5., 6.])),
                       torch.tensor([4., 10., 18.]))
    assert torch.equal(oracle.mul(torch.tensor([[1., 2.], [3., 4.]]), torch.tensor([10., 20.])),
                       torch.tensor([[10., 40.], [30., 80.]]))
    assert torch.equal(oracle.mul(torch.tensor([0., 1., 2.]), torch.tensor([0., 0., 0.])),
                       torch.zeros(3))


def test_add_relu_reference_vector():
    # tests/test_dev.py:8-18: relu(a + b) == [0, 3.6, 2.1, 0]
    a = torch.tensor([-1.5, 2.7, 1.0, 2.0])
    b = torch.tensor([-1.0, 0.9, 1.1, -2.1])
    assert torch.allclose(oracle.add_relu(a, b), torch.tensor([0, 3.6, 2.1, 0]))
    assert torch.allclose(oracle.relu(oracle.add(a, b)), torch.tensor([0, 3.6, 2.1, 0]))


def test_add_is_ieee_sum():
    # alpha = 1: the product 1*b is exact, so the result is the correctly rounded sum,
    # which is what ATen computes.  A dropped alpha or a swapped operand fails here.
    g = torch.Generator().manual_seed(11)
    a = torch.randn(4099, generator=g) * 100
    b = torch.randn(4099, generator=g) * 0.01
    assert bit_equal(oracle.add(a, b), a + b)
    special = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), float("nan"), 1e-45, 3e38])
    for x in special:
        got = oracle.add(special, x.expand(7).contiguous())
        assert ulp_diff(got, special + x) == 0


def test_add_alpha_float64_closed_form():
    # alpha != 1: two roundings; on same-sign operands (no cancellation) that is within
    # 1 ulp of the exactly rounded a + alpha*b.
    g = torch.Generator().manual_seed(12)
    a = torch.rand(10000, generator=g) + 0.5
    b = torch.rand(10000, generator=g) + 0.5
    for alpha in (0.5, 2.0, 1.7, 3.14159):
        ref = (a.double() + alpha_f32(alpha) * b.double()).float()
        assert ulp_diff(oracle.add(a, b, alpha=alpha), ref) <= 1
    # a sign error in alpha would be off by far more than 1 ulp
    assert ulp_diff(oracle.add(a, b, alpha=-1.0), a - b) == 0


def alpha_f32(alpha):
    return float(torch.tensor(alpha, dtype=torch.float32))


@pytest.mark.parametrize("ndim", [1, 2, 3, 4])
def test_index_walk_bruteforce(ndim):
    # Every permutation of the dimensions, with broadcast (size-1 expanded) operands and
    # a storage offset, against ATen on the same strided views.
    g = torch.Generator().manual_seed(100 + ndim)
    sizes = [3, 4, 2, 5][:ndim]
    for perm in itertools.permutations(range(ndim)):
        base_a = torch.randn(*sizes, generator=g)
        a = base_a.permute(*perm)
        for bc in range(1 << ndim):
            bshape = [1 if (bc >> d) & 1 else a.shape[d] for d in range(ndim)]
            store = torch.randn(7 + int(torch.tensor(bshape).prod()), generator=g)
            b = store[7:].view(*bshape)  # storage offset 7
            assert bit_equal(oracle.add(a, b), a + b)
            assert bit_equal(oracle.eq(a, b), torch.eq(a, b))
    # transposed output too
    a = torch.randn(4, 6, generator=g)
    out = torch.empty(6, 4).t()
    oracle.add(a, a, out=out)
    assert bit_equal(out.contiguous(), (a + a))


def test_relu_matches_aten_bits():
    x = torch.tensor([-0.0, 0.0, -1.0, 1.0, float("nan"), float("inf"), -float("inf"), -1e-45,
                      1e-45, -3e38])
    got = oracle.relu(x)
    ref = torch.relu(x)
    assert ulp_diff(got, ref) == 0
    assert torch.equal(torch.signbit(got), torch.signbit(ref))  # -0.0 stays -0.0
    g = torch.Generator().manual_seed(13)
    r = torch.randn(5000, generator=g)
    assert bit_equal(oracle.relu(r), torch.relu(r))
    assert bit_equal(oracle.unary(oracle.COPY, r), r)
    assert bit_equal(oracle.unary(oracle.ABS, r), r.abs())
    assert bit_equal(oracle.unary(oracle.ABS, x), x.abs())


def test_activations_against_50_digit_closed_forms():
    x, ref = load_activation_golden()
    for name, fn in (("gelu_erf", lambda t: oracle.gelu(t, "none")),
                     ("gelu_tanh", lambda t: oracle.gelu(t, "tanh")),
                     ("silu", oracle.silu)):
        ok, err, bound = rel_err_ok(fn(x), ref[name])
        worst = int(torch.argmax(err - bound))
        assert ok, f"{name}: x={x[worst].item()} err={err[worst].item()} bound={bound[worst].item()}"


def test_activation_reference_vectors():
    # tests/ops/test_gelu.py:7,18,29,43 (atol 1e-3) and test_silu.py:6,17,28,42 (atol 1e-6)
    for data in ([-1.0, 0.0, 1.0, 2.0], [[0.5, -0.5], [1.5, -1.5]], [2.0], [0.0]):
        t = torch.tensor(data, dtype=torch.float32)
        assert torch.allclose(oracle.gelu(t), F.gelu(t), atol=1e-3)
        assert torch.allclose(oracle.gelu(t, "tanh"), F.gelu(t), atol=1e-3)
        assert torch.allclose(oracle.gelu(t), F.gelu(t), atol=1e-6)  # erf form is much closer
        assert torch.allclose(oracle.silu(t), F.silu(t), atol=1e-6)


def test_gelu_distinguishes_erf_from_tanh():
    # The two formulas differ by up to 4.7e-4; the oracle must not conflate them.
    x = torch.linspace(-6, 6, 2001)
    d = (oracle.gelu(x, "none") - oracle.gelu(x, "tanh")).abs().max().item()
    assert 1e-4 < d < 1e-3


def _compare_inputs(g, n):
    a = torch.randint(0, 16, (n,), generator=g).float()
    b = torch.randint(0, 16, (n,), generator=g).float()
    a[:8] = torch.tensor([0.0, -0.0, float("nan"), float("nan"), float("inf"), 1.0, -0.0, 5.0])
    b[:8] = torch.tensor([-0.0, 0.0, float("nan"), 1.0, float("inf"), float("nan"), -0.0, 5.0])
    return a, b


def test_compare_ops_match_aten_cpu():
    g = torch.Generator().manual_seed(14)
    a, b = _compare_inputs(g, 5003)
    e = oracle.eq(a, b)
    assert e.dtype == torch.bool and bit_equal(e, torch.eq(a, b))
    assert e[0] and e[1] and not e[2] and not e[3] and e[4] and not e[5]  # IEEE: -0==+0, NaN!=NaN
    z = a.clone()
    for s in (0.0, -0.0, 5.0, float("nan")):
        n = oracle.ne_scalar(z, s)
        assert n.dtype == torch.bool and bit_equal(n, z.ne(s))
    m1, m2 = torch.eq(a, b), a.ne(0.0)
    assert bit_equal(oracle.bitwise_and(m1, m2), m1 & m2)
    # broadcast row mask
    assert bit_equal(oracle.bitwise_and(m1.view(-1, 1)[:7], m2[:5].view(1, 5)),
                     m1.view(-1, 1)[:7] & m2[:5].view(1, 5))


def test_masked_select_known_answers():
    x = torch.tensor([[0., 1., 2.], [3., 4., 5.]])
    m = torch.tensor([True, False, True])
    assert torch.equal(oracle.masked_select(x, m), torch.tensor([0., 2., 3., 5.]))
    # transposed self: order follows the logical row-major index
    xt = torch.tensor([[0., 3.], [1., 4.], [2., 5.]]).t()
    assert torch.equal(oracle.masked_select(xt, m), torch.masked_select(xt, m))
    assert torch.equal(oracle.masked_select(torch.arange(6.).view(3, 2).t(), m),
                       torch.tensor([0., 4., 1., 5.]))
    assert oracle.masked_select(x, torch.zeros(2, 3, dtype=torch.bool)).shape == (0,)
    with pytest.raises(RuntimeError):
        oracle.masked_select(x, torch.ones(2, 3))


@pytest.mark.parametrize("p", [0.0, 0.01, 0.5, 0.99, 1.0])
def test_masked_select_matches_aten_cpu(p):
    g = torch.Generator().manual_seed(15)
    x = torch.rand(20011, generator=g) * 2 - 1
    m = torch.rand(20011, generator=g) < p
    got = oracle.masked_select(x, m)
    assert bit_equal(got, torch.masked_select(x, m))
    assert got.numel() == int(m.sum())
    # broadcast in both directions
    x2 = torch.rand(37, 1, 5, generator=g)
    m2 = torch.rand(1, 11, 5, generator=g) < p
    assert bit_equal(oracle.masked_select(x2, m2), torch.masked_select(x2, m2))


def test_as_strided_admission():
    # csrc/ops/basic.cpp:254-285 against brute force over every index of the view.
    g = torch.Generator().manual_seed(16)
    for _ in range(300):
        nd = int(torch.randint(0, 4, (1,), generator=g))
        size = [int(v) for v in torch.randint(0, 4, (nd,), generator=g)]
        stride = [int(v) for v in torch.randint(-3, 5, (nd,), generator=g)]
        off = int(torch.randint(0, 6, (1,), generator=g))
        storage = int(torch.randint(0, 30, (1,), generator=g))
        numel = 1
        for s in size:
            numel *= s
        if numel == 0:
            want = 0 <= off <= storage
        else:
            idx = [off + sum(c * st for c, st in zip(coord, stride))
                   for coord in itertools.product(*[range(s) for s in size])]
            want = min(idx) >= 0 and max(idx) < storage
        assert oracle.as_strided_fits(size, stride, off, storage) == want
