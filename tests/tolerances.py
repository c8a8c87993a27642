"""Parity criteria shared by the tests.

fp32 storage : |got - ref| <= 1e-5 * max(1, |ref|)
fp16 storage : the oracle runs in fp32 on inputs already rounded to fp16 and its
               output is rounded to fp16; |got - ref16| <= max(2e-3, one fp16 ulp
               of ref16).  (Above magnitude 4 one fp16 ulp exceeds 2e-3, so a
               result that merely rounds the other way at a tie-close value cannot
               meet a pure 2e-3 bound in that storage format.)
"""
import numpy as np

F32_REL = 1e-5
F16_ABS = 2e-3


def f32_violation(got, ref):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    err = np.abs(got - ref) / np.maximum(1.0, np.abs(ref))
    return float(err.max()) if err.size else 0.0


def assert_close_f32(got, ref, rel=F32_REL, what=""):
    worst = f32_violation(got, ref)
    assert worst <= rel, "%s fp32 parity: worst |d|/max(1,|ref|) = %.3e > %.1e" % (what, worst, rel)
    return worst


def ulp16(v):
    a = np.abs(np.asarray(v, dtype=np.float64))
    e = np.floor(np.log2(np.maximum(a, 2.0 ** -14)))
    return 2.0 ** (e - 10)


def assert_close_f16(got, ref16, what=""):
    """got, ref16: float arrays holding fp16-representable values."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref16, dtype=np.float64)
    err = np.abs(got - ref)
    tol = np.maximum(F16_ABS, ulp16(ref))
    bad = err > tol
    assert not bad.any(), "%s fp16 parity: %d elements off, worst %.3e" % (what, int(bad.sum()), float(err.max()))
    exact = float((err == 0).mean()) if err.size else 1.0
    return float(err.max()) if err.size else 0.0, exact
