#!/usr/bin/env python3
"""Recipe for the polynomial inside gelu_erf_f (msd_device.h).

gelu(x) = x * Phi(x) = max(x, 0) - h(|x|),   h(t) = 0.5 * t * erfc(t / sqrt 2) = t * 2^(t * P(t) - 1)

P is the degree-7 polynomial that minimises the largest ABSOLUTE error of gelu, i.e. of h:
a weighted minimax fit of log2(erfc(t / sqrt 2)) / t on (0, 6] with weight h(t) * t * ln 2
(the sensitivity of h to an error in P), found by iteratively reweighted least squares
(Lawson's algorithm).  h is at most 0.17 and vanishes like exp(-t^2 / 2), so the tail may be
loose: the leading coefficient comes out negative, which sends 2^(t * P(t)) to zero beyond the
fitted range without any clamp on the exponent.

    python fit_gelu_poly.py            prints the eight float32 constants as they stand in msd_device.h
    python fit_gelu_poly.py --check    also compares them with the constants in msd_device.h (exit 1 on a mismatch)
"""
import os
import re
import sys

import numpy as np
from scipy import special

DEGREE = 7
T_MAX = 6.0
SAMPLES = 6000
ITERATIONS = 400


def fit(deg=DEGREE, t_max=T_MAX, n=SAMPLES, iterations=ITERATIONS):
    """-> (coefficients c0..c_deg as float64, largest absolute error of h in the model)."""
    t = np.linspace(1e-4, t_max, n)
    erfc = special.erfc(t / np.sqrt(2.0))
    target = np.log2(erfc) / t
    vander = np.vander(t / t_max, deg + 1, increasing=True)  # scaled abscissa for conditioning
    sensitivity = 0.5 * t * erfc * t * np.log(2.0)           # d h / d P
    lawson = np.ones(n)
    for _ in range(iterations):
        w = sensitivity * np.sqrt(lawson)
        coef, *_ = np.linalg.lstsq(vander * w[:, None], target * w, rcond=None)
        err = np.abs((vander @ coef - target) * sensitivity)
        lawson = lawson * (err / err.max() + 1e-3)
        lawson /= lawson.sum() / n
    return coef / t_max ** np.arange(deg + 1), float(err.max())


def gelu_float32(x, c32):
    """The float32 operation chain of gelu_erf_f emulated with numpy (each fma = one rounding)."""
    x = np.asarray(x, dtype=np.float32)
    t = np.minimum(np.abs(x), np.float32(64.0))
    t64 = t.astype(np.float64)
    p = np.full_like(t, c32[-1])
    for k in range(len(c32) - 2, -1, -1):
        p = (p.astype(np.float64) * t64 + np.float64(c32[k])).astype(np.float32)
    e = (p.astype(np.float64) * t64 - 1.0).astype(np.float32)
    with np.errstate(over="ignore", under="ignore"):
        half_erfc = np.exp2(e.astype(np.float64)).astype(np.float32)
    m = (t64 * half_erfc).astype(np.float32)
    with np.errstate(invalid="ignore"):
        s = (x.astype(np.float64) + np.abs(x).astype(np.float64)).astype(np.float32)
    return (s.astype(np.float64) * 0.5 - m.astype(np.float64)).astype(np.float32)


def header_constants(path=None):
    """The float literals of gelu_erf_f in msd_device.h, highest degree first."""
    path = path or os.path.join(os.path.dirname(os.path.abspath(__file__)), "msd_device.h")
    text = open(path).read()
    body = text[text.index("float gelu_erf_f(float x)"):]
    body = body[:body.index("\n}\n")]
    return [np.float32(v) for v in re.findall(r"(-?\d\.\d+e[+-]\d+)f", body)]


def main():
    coef, model_err = fit()
    c32 = coef.astype(np.float32)
    print("// degree %d, absolute error of the model %.2e; highest degree first" % (DEGREE, model_err))
    for c in c32[::-1]:
        print("%.9ef" % c)
    if "--check" in sys.argv:
        have = header_constants()
        want = list(c32[::-1])
        if len(have) != len(want) or any(a != b for a, b in zip(have, want)):
            print("msd_device.h holds other constants:", have)
            return 1
        print("msd_device.h matches")
    return 0


if __name__ == "__main__":
    sys.exit(main())
