"""Randomized differential test: every entry point on randomly drawn shapes, storage types,
alignments and options against the float64 oracle (fp32: 1e-5 relative; fp16 storage: the
correct rounding of a 1e-5-accurate value, half an fp16 ulp plus 1e-5 relative against the
unrounded oracle, and 2e-3 below magnitude 4; adds, permute and the DDIM update bit-exact).
The draws are seeded, so a failure names a reproducible case.  Shapes cover what the
fixed-shape tests do not: odd lengths, tiny and huge groups, batches up to 40 (launches of
many units), forced GroupNorm launch plans (workgroup size, slices, writers per unit), rows that
do not vectorise.
"""

import numpy as np
import pytest

from tolerances import ulp16

pytestmark = pytest.mark.gpu


def _bind(msd_mod, orc_mod, device, seed):
    import torch
    g = globals()
    g["msd"], g["orc"], g["dev"], g["torch"] = msd_mod, orc_mod, device, torch
    g["rng"] = np.random.default_rng(seed)


def todev(a, half):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    return t.half() if half else t


def check(name, got, ref64, half, info, scale=1.0):
    got = got.astype(np.float64)
    if half:
        err = np.abs(got - ref64)
        tol = (0.5 * ulp16(ref64) + 1e-5 * np.maximum(1.0, np.abs(ref64))) * scale
        tol = np.where(np.abs(ref64) < 4.0, np.minimum(tol, 2e-3 * scale), tol)
    else:
        err = np.abs(got - ref64); tol = 1e-5 * np.maximum(1.0, np.abs(ref64)) * scale
    bad = ~(err <= tol)
    if bad.any():
        i = np.argmax(np.where(bad, err, 0))
        print("FAIL", name, info, "half" if half else "f32", "n_bad", int(bad.sum()), "worst", float(err.flat[i]), "ref", float(ref64.flat[i]), flush=True)
        return False
    return True


def rnd_hw():
    c = rng.integers(0, 6)
    return int([rng.integers(1, 40), rng.integers(1, 5000), 8 * rng.integers(1, 600), 64, 4096, 1024][c])


def gn_case():
    groups = int(rng.choice([1, 2, 4, 8, 32])); cpg = int(rng.integers(1, 13)); C = groups * cpg
    batch = int(rng.choice([1, 2, 3, 4, 5, 6, 8, 10, 12, 17, 40])); hw = rnd_hw(); half = bool(rng.integers(0, 2)); silu = bool(rng.integers(0, 2))
    if batch * C * hw > 6e6: hw = max(1, int(6e6 // (batch * C)))
    # now and then a forced launch plan (workgroup size, slices per unit); refused values are ignored
    lib = msd.load_library()
    lib.msd_set_tuning(msd.TUNE_GN_THREADS, int(rng.choice([0, 0, 0, 64, 256, 320, 512, 640, 1024])))
    lib.msd_set_tuning(msd.TUNE_GN_SPLIT, int(rng.choice([0, 0, 0, 2, 4, 16])))
    lib.msd_set_tuning(msd.TUNE_GN_WRITERS, int(rng.choice([0, 0, 1, 2, 4, 8, 16])))  # several workgroups per whole unit
    try:
        return _gn_case(groups, cpg, C, batch, hw, half, silu)
    finally:
        lib.msd_set_tuning(msd.TUNE_GN_THREADS, 0)
        lib.msd_set_tuning(msd.TUNE_GN_SPLIT, 0)
        lib.msd_set_tuning(msd.TUNE_GN_WRITERS, 0)


def _gn_case(groups, cpg, C, batch, hw, half, silu):
    x = orc.normal((batch, C, hw), seed=int(rng.integers(1 << 30)), sigma=float(rng.uniform(0.5, 3)), mean=float(rng.uniform(-2, 2)))
    g = orc.normal((C,), seed=int(rng.integers(1 << 30)), mean=1.0, sigma=0.2); b = orc.normal((C,), seed=int(rng.integers(1 << 30)), sigma=0.2)
    eps = float(rng.choice([1e-5, 1e-6]))
    if half: x = orc.round_to_half(x)
    ref = orc.groupnorm64(x, g, b, groups, eps, silu)
    mode = int(rng.integers(0, 4)); info = (batch, C, hw, groups, silu, mode)
    xd = todev(x, half)
    if mode == 0:
        got = msd.groupnorm(xd, todev(g, 0), todev(b, 0), groups, eps, silu)
    elif mode == 1:
        got = msd.groupnorm(xd, todev(g, 0), todev(b, 0), groups, eps, silu, out=xd)
    elif mode == 2:
        if silu: ref = orc.groupnorm64(x, g, b, groups, eps, False)
        got = msd.groupnorm_tokens(xd, todev(g, 0), todev(b, 0), groups, eps).permute(0, 2, 1).contiguous()
    else:
        ch = orc.normal((batch, C), seed=int(rng.integers(1 << 30)))
        if half: ch = orc.round_to_half(ch)
        s = x + ch[:, :, None]
        if half: s = orc.round_to_half(s)
        ref = orc.groupnorm64(s.astype(np.float32), g, b, groups, eps, silu)
        got = msd.chunk_add_groupnorm(xd, todev(ch, half), todev(g, 0), todev(b, 0), groups, eps, silu)
    # tiny groups with near-zero variance amplify input rounding: scale tolerance by rstd bound
    return check("gn", got.float().cpu().numpy(), ref, half, info, scale=4.0 if cpg * hw < 16 else 1.0)


def ln_case():
    rows = int(rng.integers(1, 3000)); dim = int(rng.choice([rng.integers(1, 100), rng.integers(1, 3000), 64 * rng.integers(1, 40), 320, 640, 768, 1280]))
    if rows * dim > 4e6: rows = max(1, int(4e6 // dim))
    half = bool(rng.integers(0, 2))
    x = orc.normal((rows, dim), seed=int(rng.integers(1 << 30)), sigma=float(rng.uniform(0.5, 3)))
    g = orc.normal((dim,), seed=int(rng.integers(1 << 30)), mean=1.0, sigma=0.2); b = orc.normal((dim,), seed=int(rng.integers(1 << 30)), sigma=0.2)
    if half: x = orc.round_to_half(x)
    if dim < 4: return True
    mode = int(rng.integers(0, 3))
    if mode < 2:
        ref = orc.layernorm64(x, g, b, 1e-5); xd = todev(x, half)
        got = msd.layernorm(xd, todev(g, 0), todev(b, 0), 1e-5, out=xd if mode else None)
    else:
        r = orc.normal((rows, dim), seed=int(rng.integers(1 << 30)))
        if half: r = orc.round_to_half(r)
        s = x + r
        if half: s = orc.round_to_half(s)
        ref = orc.layernorm64(s.astype(np.float32), g, b, 1e-5)
        sm, got = msd.add_layernorm(todev(x, half), todev(r, half), todev(g, 0), todev(b, 0), 1e-5)
        if not np.array_equal(sm.float().cpu().numpy(), s.astype(np.float32)): print("FAIL add_ln sum", rows, dim, half); return False
    return check("ln", got.float().cpu().numpy(), ref, half, (rows, dim, mode))


def stream_case():
    half = bool(rng.integers(0, 2)); kind = int(rng.integers(0, 7))
    if kind == 0:
        rows = int(rng.integers(1, 600)); inner = int(rng.choice([rng.integers(1, 50), rng.integers(1, 4000), 8 * rng.integers(1, 500)]))
        ab = orc.normal((rows, 2 * inner), seed=int(rng.integers(1 << 30)), sigma=2.0)
        if half: ab = orc.round_to_half(ab)
        return check("geglu", msd.geglu(todev(ab, half)).float().cpu().numpy(), orc.geglu64(ab), half, (rows, inner))
    n = int(rng.choice([rng.integers(1, 100), rng.integers(1, 3000000)]))
    x = orc.normal((n,), seed=int(rng.integers(1 << 30)), sigma=3.0)
    if half: x = orc.round_to_half(x)
    if kind in (1, 2, 3):
        f, r = [(msd.silu, orc.silu64), (msd.gelu, orc.gelu64), (msd.quick_gelu, orc.quick_gelu64)][kind - 1]
        off = int(rng.integers(0, 2))  # unaligned view
        xd = todev(np.concatenate([[0.0], x]).astype(np.float32), half)[off:]
        xr = np.concatenate([[0.0], x]).astype(np.float32)[off:]
        return check("act%d" % kind, f(xd).float().cpu().numpy(), r(xr), half, (n, off))
    if kind == 4:
        y = orc.normal((n,), seed=int(rng.integers(1 << 30)))
        if half: y = orc.round_to_half(y)
        got = msd.elemwise_add(todev(x, half), todev(y, half)).float().cpu().numpy()
        ref = (x + y); ref = orc.round_to_half(ref) if half else ref
        ok = np.array_equal(got, ref.astype(np.float32))
        if not ok: print("FAIL add", n, half)
        return ok
    if kind == 5:
        cs = int(rng.choice([1, 3, 8, 64, 100, 4096])); nch = max(1, n // cs); n2 = nch * cs
        a = orc.normal((n2,), seed=int(rng.integers(1 << 30))); ch = orc.normal((nch,), seed=int(rng.integers(1 << 30)))
        if half: a, ch = orc.round_to_half(a), orc.round_to_half(ch)
        got = msd.chunkwise_add(todev(a, half), todev(ch, half), cs).float().cpu().numpy()
        ref = a + np.repeat(ch, cs); ref = orc.round_to_half(ref) if half else ref
        ok = np.array_equal(got, ref.astype(np.float32))
        if not ok: print("FAIL chunk add", n2, cs, half)
        return ok
    i, j, k = int(rng.integers(1, 4)), int(rng.integers(1, 700)), int(rng.integers(1, 700))
    a = orc.normal((i, j, k), seed=int(rng.integers(1 << 30)))
    if half: a = orc.round_to_half(a)
    got = msd.permute_0_2_1(todev(a, half)).float().cpu().numpy()
    ok = np.array_equal(got, a.transpose(0, 2, 1))
    if not ok: print("FAIL permute", i, j, k, half)
    return ok


def nb_case():
    half = bool(rng.integers(0, 2)); kind = int(rng.integers(0, 3))
    if kind == 0:
        rows = int(rng.integers(1, 3000)); cols = int(rng.choice([rng.integers(1, 200), rng.integers(1, 9000), 77, 64, 256, 1024, 4096]))
        if rows * cols > 4e6: rows = max(1, int(4e6 // cols))
        x = orc.normal((rows, cols), seed=int(rng.integers(1 << 30)), sigma=float(rng.uniform(0.5, 4)))
        if half: x = orc.round_to_half(x)
        stable = bool(rng.integers(0, 2)); xd = todev(x, half)
        got = msd.softmax(xd, stable=stable, out=xd if rng.integers(0, 2) else None).float().cpu().numpy().astype(np.float64)
        ref = orc.softmax64(x)
        if half:
            ref16 = orc.round_to_half(ref.astype(np.float32)).astype(np.float64)
            ok = bool((np.abs(got - ref16) <= ulp16(ref16)).all())
        else:
            ok = bool((np.abs(got - ref) <= 1e-5 * ref + 1e-12).all())
        if not ok: print("FAIL softmax", rows, cols, half, stable, flush=True)
        return ok
    if kind == 1:
        m = int(rng.integers(1, 9)); n = int(rng.integers(1, 1500)); k = int(rng.choice([rng.integers(1, 100), rng.integers(1, 3000), 320, 1280, 8 * rng.integers(1, 300)]))
        x = orc.normal((m, k), seed=int(rng.integers(1 << 30))); w = orc.normal((n, k), seed=int(rng.integers(1 << 30)), sigma=k ** -0.5)
        b = orc.normal((n,), seed=int(rng.integers(1 << 30)), sigma=0.1) if rng.integers(0, 2) else None
        if half: x, w = orc.round_to_half(x), orc.round_to_half(w)
        ai, ao = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        xin = orc.silu64(x).astype(np.float32) if ai else x
        ref = orc.linear64(xin, w, b)
        if ao: ref = ref / (1 + np.exp(-ref))
        got = msd.linear_rows(todev(x, half), todev(w, half), todev(b, 0) if b is not None else None, ai, ao)
        return check("linear", got.float().cpu().numpy(), ref, half, (m, n, k, ai, ao))
    n = int(rng.choice([rng.integers(1, 100), rng.integers(1, 200000)]))
    x = orc.normal((n,), seed=int(rng.integers(1 << 30))); e = orc.normal((n,), seed=int(rng.integers(1 << 30)))
    ts, a, ap, s1m = orc.ddim_schedule(int(rng.choice([50, 25, 10])))
    i = int(rng.integers(0, len(ts)))
    got = msd.ddim_update(todev(x, 0), todev(e, 0), float(a[i]), float(ap[i]), float(s1m[i])).cpu().numpy()
    ok = np.array_equal(got, orc.ddim_update(x, e, a[i], ap[i], s1m[i]))
    if not ok: print("FAIL ddim", n, i)
    return ok



@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_shapes_against_float64_oracle(msd, orc, cuda, seed):
    _bind(msd, orc, cuda, seed)
    cases = [gn_case, gn_case, ln_case, stream_case, nb_case]
    failures = 0
    for _ in range(300):
        failures += 0 if cases[int(rng.integers(0, len(cases)))]() else 1
    assert failures == 0, "%d random cases failed (details printed above)" % failures
    assert msd.status() == 0
