"""Helpers shared by the tests: ulp distance, tolerances, golden vectors."""
import json
import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

# Tolerance of the activation kernels and of the oracle against the closed form:
# |got - ref| <= 2e-6 * |ref| + ABS_FLOOR.  The floor is four subnormal steps
# (2^-149 each): it only matters where x*Phi(x) itself is subnormal.
REL_TOL = 2e-6
ABS_FLOOR = 4 * 2.0 ** -149
# The tanh form of GeLU is not a headline op (the reference's own test holds it to
# atol 1e-3): its exponent argument 2u is rounded to binary32, which costs
# |2u| * 2^-24 of relative error, i.e. more than 2e-6 once |x| > 5, where the value
# itself is below 2e-7.  An absolute floor of 1e-10 covers that tail.
FLOOR = {"gelu_erf": ABS_FLOOR, "silu": ABS_FLOOR, "gelu_tanh": 1e-10}


def ordered_int(t):
    """Map float32 bit patterns to integers that are monotone in the float value
    (so that |difference| is the distance in ulps); +0 and -0 map to the same value."""
    i = t.contiguous().view(torch.int32).to(torch.int64)
    return torch.where(i < 0, -(i & 0x7FFFFFFF), i)


def ulp_diff(a, b):
    """Largest distance in float32 ulps between two float32 tensors.  NaNs must sit
    in the same places."""
    assert a.dtype == torch.float32 and b.dtype == torch.float32 and a.shape == b.shape
    na, nb = torch.isnan(a), torch.isnan(b)
    assert torch.equal(na, nb), "NaN pattern differs"
    if a.numel() == 0:
        return 0
    d = (ordered_int(a) - ordered_int(b)).abs()
    d = torch.where(na, torch.zeros_like(d), d)
    return int(d.max().item())


def bit_equal(a, b):
    """True if two tensors have identical shapes, dtypes and bytes."""
    if a.shape != b.shape or a.dtype != b.dtype:
        return False
    if a.numel() == 0:
        return True
    # copy into fresh 1-D tensors: a "contiguous" tensor may still carry odd strides on
    # size-1 dimensions, which view(dtype) refuses
    av = torch.empty(a.numel(), dtype=a.dtype).copy_(a.reshape(-1)).view(torch.uint8)
    bv = torch.empty(b.numel(), dtype=b.dtype).copy_(b.reshape(-1)).view(torch.uint8)
    return bool(torch.equal(av, bv))


def rel_err_ok(got, ref64, rel=REL_TOL, floor=ABS_FLOOR):
    """got: float32 tensor, ref64: float64 tensor of the closed form."""
    g = got.to(torch.float64)
    err = (g - ref64).abs()
    bound = rel * ref64.abs() + floor
    bad = err > bound
    # NaN in the reference (inputs +-inf) must be NaN in the result
    nan_ref = torch.isnan(ref64)
    bad = torch.where(nan_ref, ~torch.isnan(g), bad)
    return not bool(bad.any()), err, bound


def closed_form64(name, x):
    """Closed forms in float64 (scipy), used for large random inputs where the
    50-digit fixtures do not reach.  x: float32 tensor."""
    from scipy import special
    xd = x.to(torch.float64).numpy()
    if name == "gelu_erf":
        r = 0.5 * xd * special.erfc(-xd / np.sqrt(2.0))
    elif name == "gelu_tanh":
        u = np.sqrt(2.0 / np.pi) * (xd + 0.044715 * xd ** 3)
        with np.errstate(over="ignore"):
            r = xd / (1.0 + np.exp(-2.0 * u))
    elif name == "silu":
        with np.errstate(over="ignore"):
            r = xd / (1.0 + np.exp(-xd))
    else:
        raise KeyError(name)
    return torch.from_numpy(np.asarray(r))


def load_activation_golden():
    with open(os.path.join(GOLDEN, "activations_mp.json")) as f:
        rows = json.load(f)["points"]
    bits = np.array([r["x_bits"] for r in rows], dtype=np.uint32)
    x = torch.from_numpy(bits.view(np.float32).copy())
    ref = {k: torch.tensor([float(r[k]) for r in rows], dtype=torch.float64)
           for k in ("gelu_erf", "gelu_tanh", "silu")}
    return x, ref
