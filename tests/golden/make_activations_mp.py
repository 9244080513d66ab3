#!/usr/bin/env python3
"""Writes activations_mp.json: closed-form values of gelu (erf and tanh forms) and
silu at 50 significant digits (mpmath), for float32 inputs given by bit pattern.

These vectors pin the CPU oracle (oracle/twg_oracle.c) and, through it, the HIP
kernels.  Nothing from the reference is executed: the formulas are
  gelu 'none' : x * Phi(x)                      (ATen's definition of exact GeLU)
  gelu 'tanh' : 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))   csrc/ops/unary.cpp:94
  silu        : x / (1 + exp(-x))                                  csrc/ops/unary.cpp:97
Run:  python tests/golden/make_activations_mp.py
"""
import json
import os
import struct

import mpmath as mp
import numpy as np

mp.mp.dps = 50


def f32(x):
    return struct.unpack("<f", struct.pack("<f", float(x)))[0]


def bits(x):
    return struct.unpack("<I", struct.pack("<f", float(x)))[0]


def points():
    pts = [0.0, -0.0, 1e-30, -1e-30, 1e-45, -1e-45, 1e-40, -1e-40, 1.1754944e-38, -1.1754944e-38]
    # inputs of the reference's own tests (tests/ops/test_gelu.py, test_silu.py, test_add.py)
    pts += [-1.0, 0.0, 1.0, 2.0, 0.5, -0.5, 1.5, -1.5, -2.5, 3.6, 2.1, -0.1]
    pts += list(np.arange(-14.0, 14.01, 0.25))
    pts += [18.7, -18.7, 5.5, -5.5, 6.0, -6.0, 13.0, -13.0, -13.06, -13.9, -14.2, 20.0, -20.0,
            50.0, -50.0, 80.0, -80.0, 87.0, -87.0, 88.0, -88.0, 100.0, -100.0]
    rng = np.random.default_rng(20240607)
    pts += list(rng.normal(0.0, 3.0, 200))
    pts += list(rng.uniform(-4.0, 4.0, 100))
    seen, out = set(), []
    for p in pts:
        b = bits(p)
        if b not in seen:
            seen.add(b)
            out.append(f32(p))
    return out


def gelu_erf(x):
    return x * mp.ncdf(x)


def gelu_tanh(x):
    u = mp.sqrt(2 / mp.pi) * (x + mp.mpf("0.044715") * x ** 3)
    return x / (1 + mp.exp(-2 * u))


def silu(x):
    return x / (1 + mp.exp(-x))


def main():
    rows = []
    for p in points():
        x = mp.mpf(p)  # exact value of the float32 input
        rows.append({
            "x_bits": bits(p),
            "x": repr(p),
            # 25 significant digits: far beyond binary64, parsed with float()
            "gelu_erf": mp.nstr(gelu_erf(x), 25),
            "gelu_tanh": mp.nstr(gelu_tanh(x), 25),
            "silu": mp.nstr(silu(x), 25),
        })
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "activations_mp.json"), "w") as f:
        json.dump({"digits": 50, "points": rows}, f, indent=0)
    print(len(rows), "points")


if __name__ == "__main__":
    main()
