"""The polynomial inside the device GELU (csrc/msd_device.h: gelu_erf_f) is reproducible and as
accurate as its comment says: the recipe next to it regenerates the committed constants, and the
float32 operation chain of the device function, emulated in numpy, stays within 2.5e-7 of
float64 erfc-based GELU.  (The reference evaluates x * 0.5 * (1 + erf(x * M_SQRT1_2_F)),
K/util.cl:104-122; the oracle restates that with erff and is what the GPU tests compare with.)"""
import importlib.util
import os

import numpy as np
from scipy import special

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
RECIPE = os.path.join(REPO, "mobile-stable-diffusion_amd", "csrc", "fit_gelu_poly.py")


def _recipe():
    spec = importlib.util.spec_from_file_location("fit_gelu_poly", RECIPE)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _gelu64(x):
    x = np.asarray(x, dtype=np.float64)
    return 0.5 * x * special.erfc(-x / np.sqrt(2.0))


def test_recipe_regenerates_the_committed_constants():
    r = _recipe()
    coef, model_err = r.fit()
    have = r.header_constants()
    want = list(coef.astype(np.float32)[::-1])
    assert len(have) == r.DEGREE + 1 == 8
    assert [float(v) for v in have] == [float(v) for v in want]  # the same float32 values
    for h, c in zip(have, coef[::-1]):  # and the float64 fit is what they round
        assert abs(float(h) - c) <= 1e-6 * abs(c)
    assert model_err < 1e-8  # the polynomial itself costs 9e-9 absolute; the rest is float32 rounding
    assert coef[-1] < 0     # the power of two dies out beyond the fitted range


def test_float32_chain_is_within_its_stated_error_of_float64():
    r = _recipe()
    c32 = np.array(r.header_constants()[::-1], dtype=np.float32)
    x = np.concatenate([np.linspace(-12.0, 12.0, 2400001), np.linspace(-70.0, 70.0, 140001),
                        np.array([0.0, 1e-30, -1e-30, 1e-3, -1e-3, 88.0, -88.0, 1e30, -1e30])]).astype(np.float32)
    got = r.gelu_float32(x, c32)
    ref = _gelu64(x)
    err = np.abs(got.astype(np.float64) - ref)
    assert err.max() <= 2.5e-7, "worst %.3e at %r" % (err.max(), float(x[err.argmax()]))
    assert (err / np.maximum(1.0, np.abs(ref))).max() <= 1.0e-7
    # the expression the reference evaluates, in float32, is no closer to float64
    x32 = x[np.abs(x) <= 12]
    erff = special.erf((x32 * np.float32(0.70710678)).astype(np.float32)).astype(np.float32)
    formula = x32 * np.float32(0.5) * (np.float32(1.0) + erff)
    assert np.abs(formula.astype(np.float64) - _gelu64(x32)).max() >= 2.5e-7
    # special values: zero, signed infinities, NaN, and no negative zero surprises
    s = r.gelu_float32(np.array([0.0, 100.0, -100.0, np.inf, 30.0, -30.0], dtype=np.float32), c32)
    assert s[0] == 0 and s[1] == 100.0 and abs(s[2]) < 1e-30 and s[3] == np.inf and s[4] == 30.0 and abs(s[5]) < 1e-30
    assert np.isnan(r.gelu_float32(np.array([np.nan], dtype=np.float32), c32))[0]
    # symmetry gelu(x) - gelu(-x) = x holds to rounding
    xs = np.linspace(0.0, 8.0, 80001).astype(np.float32)
    d = r.gelu_float32(xs, c32).astype(np.float64) - r.gelu_float32(-xs, c32).astype(np.float64)
    assert np.abs(d - xs).max() <= 5e-7
