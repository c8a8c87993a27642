"""Parity criteria shared by the tests.

fp32 storage : |got - ref| <= 1e-5 * max(1, |ref|)
fp16 storage : the oracle runs in fp32 on inputs already rounded to fp16; its UNROUNDED fp32
               output `ref32` is the reference.  A stored fp16 value must be the correct
               rounding of a value that is 1e-5-accurate:
                   |got - ref32| <= 0.5 * ulp16(ref32) + 1e-5 * max(1, |ref32|)
               everywhere, and |got - ref32| <= 2e-3 wherever |ref32| < 4 (above 4 half an
               fp16 ulp alone reaches 2e-3, so no fp16 storage can promise it there).  This
               rejects truncation, a wrong rounding mode and a value that is a whole ulp off.

Every fp16 check also records, per label, the worst error and how many elements exceed a bare
2e-3 (all of them sit above |ref32| = 4 if the assertion held); at the end of a GPU run
conftest.py writes the table as parity_fp16.json into the run's output folder.
"""
import numpy as np

F32_REL = 1e-5
F16_ABS = 2e-3

# label -> dict(n, worst, over_2e3, budget_used, exact) filled by assert_close_f16
FP16_REPORT = {}


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
    """Spacing of IEEE binary16 at |v| (the subnormal spacing 2^-24 below 2^-14)."""
    a = np.abs(np.asarray(v, dtype=np.float64))
    e = np.floor(np.log2(np.maximum(a, 2.0 ** -14)))
    return 2.0 ** (e - 10)


def assert_close_f16(got, ref32, what="", rel_floor=1.0):
    """got: fp16-representable values (any float dtype); ref32: the oracle's unrounded output.
    rel_floor: the 1e-5 term is relative to max(rel_floor, |ref32|); 0 makes it purely relative.
    Returns (worst absolute error, fraction of elements equal to the correctly rounded ref32)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref32, dtype=np.float64)
    assert got.shape == ref.shape, "%s: shape %s vs %s" % (what, got.shape, ref.shape)
    err = np.abs(got - ref)
    aref = np.abs(ref)
    half_ulp = 0.5 * ulp16(ref)
    tol = half_ulp + F32_REL * np.maximum(rel_floor, aref)
    bad = err > tol
    small = aref < 4.0
    bad_small = small & (err > F16_ABS)
    worst = float(err.max()) if err.size else 0.0
    with np.errstate(over="ignore"):
        rounded = np.asarray(ref32, dtype=np.float32).astype(np.float16).astype(np.float64)
    exact = float((got == rounded).mean()) if err.size else 1.0
    if what:
        rec = FP16_REPORT.setdefault(what, {"n": 0, "worst": 0.0, "over_2e3": 0, "budget_used": 0.0,
                                            "exact": 1.0})
        rec["n"] += int(err.size)
        rec["worst"] = max(rec["worst"], worst)
        rec["over_2e3"] += int((err > F16_ABS).sum())
        if err.size:  # share of the 1e-5 allowance that the worst element needs beyond half an ulp
            rec["budget_used"] = max(rec["budget_used"],
                                     float(((err - half_ulp) / (F32_REL * np.maximum(rel_floor, aref) + 1e-300)).max()))
        rec["exact"] = min(rec["exact"], exact)
    assert not bad.any(), "%s fp16 parity: %d elements beyond half an ulp + 1e-5, worst %.3e at ref %.6g" % (
        what, int(bad.sum()), float(err[bad].max()), float(ref[bad][np.argmax(err[bad])]))
    assert not bad_small.any(), "%s fp16 parity: %d elements with |ref| < 4 off by more than 2e-3" % (
        what, int(bad_small.sum()))
    return worst, exact


def assert_one_ulp16_apart(a, b, what=""):
    """Two fp16 results of the same quantity by different routes (each a correct rounding of a
    1e-5-accurate value) may differ by one fp16 ulp where that value sits next to a rounding
    boundary, never by more."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    err = np.abs(a - b)
    tol = np.maximum(ulp16(a), ulp16(b))
    bad = err > tol
    assert not bad.any(), "%s: %d elements more than one fp16 ulp apart, worst %.3e" % (
        what, int(bad.sum()), float(err.max()))
    return float((err == 0).mean()) if err.size else 1.0
