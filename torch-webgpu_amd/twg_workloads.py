"""Seeded synthetic inputs for the five benchmark configurations, on the host.

Shared by bench.py (full size) and the parity tests (reduced size): the same
generator code, so the tests exercise the value distributions the benchmark
times.  Every function returns CPU tensors; `n` is the element count
(2**28 in the benchmark).
"""
import math

import torch


def _gen(seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def add_contiguous(n=1 << 20, seed=0):
    """Config 1: two contiguous fp32 vectors, uniform in [-4, 4)."""
    g = _gen(seed)
    a = torch.rand(n, generator=g, dtype=torch.float32) * 8.0 - 4.0
    b = torch.rand(n, generator=g, dtype=torch.float32) * 8.0 - 4.0
    return a, b


def activation_input(rows=16384, cols=16384, seed=1):
    """Config 2: N(0, 3^2) with 0.1% of the entries forced, in equal thirds, to
    0.0, +1e-30 and -1e-30."""
    g = _gen(seed)
    x = torch.randn(rows * cols, generator=g, dtype=torch.float32) * 3.0
    m = max(3, (rows * cols) // 1000)
    idx = torch.randint(0, rows * cols, (m,), generator=g)
    third = m // 3
    x[idx[:third]] = 0.0
    x[idx[third:2 * third]] = 1e-30
    x[idx[2 * third:]] = -1e-30
    return x.view(rows, cols)


def broadcast_add_inputs(rows=8192, cols=32768, seed=2):
    """Config 3: A[rows, cols], bias[1, cols] and C[cols, rows], uniform in [-1, 1).
    3a is A + bias; 3b is A viewed as (cols, rows) with strides (1, cols) plus C."""
    g = _gen(seed)
    a = torch.rand(rows, cols, generator=g, dtype=torch.float32) * 2.0 - 1.0
    bias = torch.rand(1, cols, generator=g, dtype=torch.float32) * 2.0 - 1.0
    c = torch.rand(cols, rows, generator=g, dtype=torch.float32) * 2.0 - 1.0
    return a, bias, c


def mask_inputs(n=1 << 28, seed=3):
    """Config 4: two integer-valued fp32 tensors in {0..15} (about 1/16 equal) and an
    fp32 tensor that is 30% exact zeros."""
    g = _gen(seed)
    p = torch.randint(0, 16, (n,), generator=g, dtype=torch.int32).to(torch.float32)
    q = torch.randint(0, 16, (n,), generator=g, dtype=torch.int32).to(torch.float32)
    z = torch.rand(n, generator=g, dtype=torch.float32) * 2.0 - 1.0
    z[z == 0.0] = 0.5  # keep the zero fraction exactly the Bernoulli one
    zero = torch.rand(n, generator=g, dtype=torch.float32) < 0.3
    z[zero] = 0.0
    return p, q, z


def select_source(n=1 << 28, seed=4):
    """Config 5 source: uniform in [-1, 1)."""
    g = _gen(seed)
    return torch.rand(n, generator=g, dtype=torch.float32) * 2.0 - 1.0


def bernoulli_mask(n, p, seed=5):
    """Config 5 mask: independent Bernoulli(p) per element."""
    g = _gen(seed + int(round(p * 1000)))
    return torch.rand(n, generator=g, dtype=torch.float32) < p


def alternating_density_mask(n, span=8192, p_lo=0.01, p_hi=0.9, seed=7):
    """Spans of `span` elements that alternate between Bernoulli(p_lo) and Bernoulli(p_hi):
    with span = 8192 (one wavefront's share of a masked_select tile) neighbouring
    wavefronts of one tile take the gather path and the streaming loop in turn."""
    g = _gen(seed)
    u = torch.rand(n, generator=g, dtype=torch.float32)
    hi = (torch.arange(n, dtype=torch.int64) // span) % 2 == 1
    return torch.where(hi, u < p_hi, u < p_lo)


def clustered_mask(n, mean_run=4096, seed=6):
    """Config 5 clustered mask: alternating runs of true/false whose lengths are
    geometric with the given mean."""
    g = _gen(seed)
    p = 1.0 / mean_run
    out = torch.empty(n, dtype=torch.bool)
    filled = 0
    value = True
    while filled < n:
        k = max(16, int((n - filled) / mean_run * 1.2) + 16)
        u = torch.rand(k, generator=g, dtype=torch.float64).clamp_(min=1e-300)
        runs = torch.floor(torch.log(u) / math.log1p(-p)).to(torch.int64) + 1
        ends = torch.cumsum(runs, 0)
        keep = int((ends <= n - filled).sum().item())
        if keep < k:
            keep += 1  # the run that crosses the end is cut short
        runs = runs[:keep]
        vals = torch.zeros(keep, dtype=torch.bool)
        vals[(0 if value else 1)::2] = True
        seg = torch.repeat_interleave(vals, runs)
        take = min(seg.numel(), n - filled)
        out[filled:filled + take] = seg[:take]
        filled += take
        if keep % 2 == 1:
            value = not value
    return out


# Algorithmic bytes per element (what bandwidth figures are computed from).
BYTES_PER_ELEM = {
    "add": 12, "gelu": 8, "silu": 8, "relu": 8, "add_rowbias": 8, "add_transposed": 12,
    "eq": 9, "ne_scalar": 5, "bitwise_and": 3,
}


def masked_select_bytes(n, k):
    """Source (4 B) and mask (1 B) read once, k selected values written."""
    return 5 * n + 4 * k
