"""Parity of the path's neighbours (through the C ABI) against the CPU oracle:
the Linear layers of the time embedding, the row softmax, the DDIM schedule and
update.  Same criteria as test_gpu_parity.py; the DDIM update and everything
integer is bit-exact.
"""
import numpy as np
import pytest

from tolerances import assert_close_f16, assert_close_f32

pytestmark = pytest.mark.gpu


def _torch():
    import torch
    return torch


def _to_dev(a, cuda, half=False):
    t = _torch().from_numpy(np.ascontiguousarray(a)).to(cuda)
    return t.half() if half else t


# ----------------------------------------------------------------- Linear on embedding rows
def _linear_case(msd, orc, cuda, m, n, k, seed, half, act_in=0, act_out=0, bias=True):
    x = orc.normal((m, k), seed=seed)
    w = orc.normal((n, k), seed=seed + 1, sigma=1.0 / np.sqrt(k))
    b = orc.normal((n,), seed=seed + 2, sigma=0.1) if bias else None
    if half:
        x, w = orc.round_to_half(x), orc.round_to_half(w)
    xin = orc.silu(x) if act_in else x
    ref = orc.linear(xin, w, b)
    ref64 = orc.linear64(xin, w, b)
    if act_out:
        ref, ref64 = orc.silu(ref), orc.silu64(ref64.astype(np.float32))
    got = msd.linear_rows(_to_dev(x, cuda, half), _to_dev(w, cuda, half),
                          _to_dev(b, cuda) if bias else None, act_in, act_out).float().cpu().numpy()
    what = "linear m%d n%d k%d" % (m, n, k)
    if half:
        worst, exact = assert_close_f16(got, ref, what)
        return exact
    assert_close_f32(got, ref, what=what)
    if not act_out:
        assert_close_f32(got, ref64, 3e-6, what + " vs f64")
    return None


@pytest.mark.parametrize("name", ["lin_a", "lin_b", "lin_c"])
def test_linear_library_fixtures(msd, cuda, golden, name):
    x, w = golden[name + "_x"], golden[name + "_w"]
    b = _to_dev(golden[name + "_b"], cuda) if name + "_b" in golden.files else None
    xd, wd = _to_dev(x, cuda), _to_dev(w, cuda)
    assert_close_f32(msd.linear_rows(xd, wd, b).cpu().numpy(), golden[name + "_y"], what=name)
    assert_close_f32(msd.linear_rows(xd, wd, b, act_in=msd.ACT_SILU).cpu().numpy(),
                     golden[name + "_y_silu_in"], what=name + " silu in")
    assert_close_f32(msd.linear_rows(xd, wd, b, act_out=msd.ACT_SILU).cpu().numpy(),
                     golden[name + "_y_silu_out"], what=name + " silu out")


# time_embed_0 (320 -> 1280, SiLU behind it), time_embed_2 (1280 -> 1280), and the per-ResBlock
# SiLU(emb) -> Linear(1280 -> Cout) for Cout = 320 / 640 / 1280
@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
@pytest.mark.parametrize("n,k,act_in,act_out", [(1280, 320, 0, 1), (1280, 1280, 0, 0), (320, 1280, 1, 0),
                                                (640, 1280, 1, 0), (1280, 1280, 1, 0)])
def test_linear_time_embedding_shapes(msd, orc, cuda, n, k, act_in, act_out, half):
    exact = _linear_case(msd, orc, cuda, 2, n, k, 7000 + n + k, half, act_in, act_out)
    if half:
        assert exact > 0.99


@pytest.mark.parametrize("m,n,k", [(1, 64, 320), (3, 33, 96), (5, 7, 1280), (8, 130, 1280), (8, 16, 2048),
                                   (2, 5, 77), (4, 9, 1), (2, 3, 8), (7, 1, 40)])
def test_linear_edge_shapes(msd, orc, cuda, m, n, k):
    _linear_case(msd, orc, cuda, m, n, k, 7100 + m * 1000 + n + k, False)
    _linear_case(msd, orc, cuda, m, n, k, 7200 + m * 1000 + n + k, True, act_in=1, bias=False)


def test_linear_unaligned_views_and_rejections(msd, orc, cuda):
    torch = _torch()
    x = orc.normal((2, 328), seed=7301)
    w = orc.normal((20, 328), seed=7302, sigma=0.05)
    big = _to_dev(np.concatenate([[0.0], w.reshape(-1)]).astype(np.float32), cuda)
    wd = big[1:].view(20, 328)  # 4 bytes past a 16-byte boundary
    got = msd.linear_rows(_to_dev(x, cuda), wd).cpu().numpy()
    assert_close_f32(got, orc.linear(x, w), what="unaligned weight")
    lib = msd.load_library()
    xd = _to_dev(x, cuda)
    s = torch.cuda.current_stream().cuda_stream
    assert lib.msd_linear_rows(xd.data_ptr(), wd.data_ptr(), None, xd.data_ptr(), 2, 20, 328, 0, 0, 0, s) == 1
    nine = torch.zeros((9, 328), device=cuda)
    out = torch.zeros((9, 20), device=cuda)
    assert lib.msd_linear_rows(nine.data_ptr(), wd.data_ptr(), None, out.data_ptr(), 9, 20, 328, 0, 0, 0, s) == 1
    assert lib.msd_linear_rows(xd.data_ptr(), wd.data_ptr(), None, out.data_ptr(), 2, 20, 328, 2, 0, 0, s) == 1
    assert lib.msd_linear_rows(xd.data_ptr(), wd.data_ptr(), None, out.data_ptr(), 0, 20, 328, 0, 0, 0, s) == 0


# output channels of the 22 ResBlocks of one UNet step, in execution order (M/UNetModel.cpp:86-1018)
RESBLOCK_COUT = [320, 320, 640, 640, 1280, 1280, 1280, 1280, 1280, 1280, 1280, 1280, 1280, 1280, 1280, 1280,
                 640, 640, 640, 320, 320, 320]


@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
def test_grouped_linear_runs_the_22_resblock_projections_in_one_launch(msd, orc, cuda, half):
    """SiLU(emb) -> Linear(1280 -> Cout) of every ResBlock (M/nn/ResBlock.cpp:173-183) as one
    launch: each output against the oracle and bit for bit against its own msd_linear_rows call."""
    torch = _torch()
    emb = orc.normal((2, 1280), seed=7500, sigma=1.5)
    ws = [orc.normal((n, 1280), seed=7501 + i, sigma=1280 ** -0.5) for i, n in enumerate(RESBLOCK_COUT)]
    bs = [orc.normal((n,), seed=7601 + i, sigma=0.1) for i, n in enumerate(RESBLOCK_COUT)]
    if half:
        emb, ws = orc.round_to_half(emb), [orc.round_to_half(w) for w in ws]
    ed = _to_dev(emb, cuda, half)
    wd = [_to_dev(w, cuda, half) for w in ws]
    bd = [_to_dev(b, cuda) for b in bs]
    outs = msd.linear_rows_grouped(ed, wd, bd, act_in=msd.ACT_SILU)
    assert len(outs) == 22
    for i, (o, w, b) in enumerate(zip(outs, ws, bs)):
        single = msd.linear_rows(ed, wd[i], bd[i], act_in=msd.ACT_SILU)
        assert torch.equal(o, single), "problem %d differs from its own launch" % i
        ref = orc.linear(orc.silu(emb), w, b)
        if half:
            assert_close_f16(o.float().cpu().numpy(), ref, "grouped linear f16")
        else:
            assert_close_f32(o.cpu().numpy(), ref, what="grouped linear %d" % i)


def test_grouped_linear_edge_cases(msd, orc, cuda):
    torch = _torch()
    # more problems than one launch's table holds, empty problems, missing biases, no activation
    ns = [3, 0, 130, 1, 64] * 8
    x = orc.normal((3, 96), seed=7700)
    ws = [orc.normal((n, 96), seed=7701 + i, sigma=0.1) for i, n in enumerate(ns)]
    bs = [orc.normal((n,), seed=7801 + i) if i % 3 else None for i, n in enumerate(ns)]
    xd = _to_dev(x, cuda)
    outs = msd.linear_rows_grouped(xd, [_to_dev(w, cuda) for w in ws],
                                   [_to_dev(b, cuda) if b is not None else None for b in bs], act_out=msd.ACT_SILU)
    for o, w, b, n in zip(outs, ws, bs, ns):
        assert o.shape == (3, n)
        if n:
            assert_close_f32(o.cpu().numpy(), orc.silu(orc.linear(x, w, b)), what="grouped edge")
    # k that does not vectorise: falls back to one scalar launch per problem, same results
    x2 = orc.normal((2, 77), seed=7900)
    w2 = [orc.normal((5, 77), seed=7901), orc.normal((9, 77), seed=7902)]
    o2 = msd.linear_rows_grouped(_to_dev(x2, cuda), [_to_dev(w, cuda) for w in w2])
    for o, w in zip(o2, w2):
        assert_close_f32(o.cpu().numpy(), orc.linear(x2, w), what="grouped odd k")
    assert msd.linear_rows_grouped(xd, []) == []
    # rejections: more than 8 rows, an output that is the input
    lib = msd.load_library()
    import ctypes
    vp = ctypes.c_void_p
    arr = lambda *v: (vp * len(v))(*v)
    one = (ctypes.c_size_t * 1)(96)
    s = torch.cuda.current_stream().cuda_stream
    wdev = _to_dev(ws[2], cuda)
    assert lib.msd_linear_rows_grouped(xd.data_ptr(), arr(wdev.data_ptr()), None, arr(xd.data_ptr()), one, 1, 3, 96,
                                       0, 0, 0, s) == 1
    assert lib.msd_linear_rows_grouped(xd.data_ptr(), arr(wdev.data_ptr()), None, arr(outs[2].data_ptr()), one, 1, 9,
                                       96, 0, 0, 0, s) == 1


def test_time_embedding_mlp_chain(msd, orc, cuda):
    """timestep -> sinusoid -> Linear+SiLU -> Linear -> SiLU+Linear, as one UNet step runs it."""
    torch = _torch()
    t = np.array([981, 961], dtype=np.int64)
    w0 = orc.normal((1280, 320), seed=7401, sigma=320 ** -0.5)
    b0 = orc.normal((1280,), seed=7402, sigma=0.1)
    w2 = orc.normal((1280, 1280), seed=7403, sigma=1280 ** -0.5)
    b2 = orc.normal((1280,), seed=7404, sigma=0.1)
    we = orc.normal((640, 1280), seed=7405, sigma=1280 ** -0.5)
    be = orc.normal((640,), seed=7406, sigma=0.1)
    temb = np.stack([orc.timestep_embedding(int(v)) for v in t])
    h = orc.silu(orc.linear(temb, w0, b0))
    emb = orc.linear(h, w2, b2)
    ref = orc.linear(orc.silu(emb), we, be)
    d = lambda a: _to_dev(a, cuda)
    temb_d = msd.timestep_embedding(torch.from_numpy(t).to(cuda), 320)
    h_d = msd.linear_rows(temb_d, d(w0), d(b0), act_out=msd.ACT_SILU)
    emb_d = msd.linear_rows(h_d, d(w2), d(b2))
    out_d = msd.linear_rows(emb_d, d(we), d(be), act_in=msd.ACT_SILU)
    assert_close_f32(emb_d.cpu().numpy(), emb, what="time_embed")
    assert_close_f32(out_d.cpu().numpy(), ref, what="resblock emb projection")


# ----------------------------------------------------------------- softmax
def _softmax_case(msd, orc, cuda, rows, cols, seed, half, stable, sigma=2.0, inplace=False):
    x = orc.normal((rows, cols), seed=seed, sigma=sigma)
    if half:
        x = orc.round_to_half(x)
    ref = orc.softmax(x)
    xd = _to_dev(x, cuda, half)
    got = msd.softmax(xd, stable=stable, out=xd if inplace else None).float().cpu().numpy()
    what = "softmax %dx%d stable=%d" % (rows, cols, stable)
    if half:
        # probabilities are far below the 2e-3 absolute criterion: the stored value must be the
        # correct fp16 rounding of a value within 1e-5 RELATIVE of the oracle's
        worst, exact = assert_close_f16(got, ref, what, rel_floor=0.0)
        assert exact > 0.99, what
    else:
        assert_close_f32(got, ref, what=what)
        np.testing.assert_allclose(got, orc.softmax64(x), rtol=1e-5, atol=1e-9)
        np.testing.assert_allclose(got.astype(np.float64).sum(axis=-1), 1.0, atol=1e-5)


@pytest.mark.parametrize("stable", [0, 1])
@pytest.mark.parametrize("name", ["sm_a", "sm_b", "sm_c"])
def test_softmax_library_fixtures(msd, cuda, golden, name, stable):
    got = msd.softmax(_to_dev(golden[name + "_x"], cuda), stable=stable).cpu().numpy()
    assert_close_f32(got, golden[name + "_y"], what=name)
    np.testing.assert_allclose(got, golden[name + "_y"], rtol=1e-5, atol=1e-9)


# self-attention rows of the UNet (keys = 4096 / 1024 / 256 / 64 latent tokens) and the
# cross-attention rows (77 text tokens); rows cut down, the row length is what dispatches
@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
@pytest.mark.parametrize("stable", [0, 1])
@pytest.mark.parametrize("rows,cols", [(96, 4096), (130, 1024), (257, 256), (301, 64), (1000, 77)])
def test_softmax_attention_shapes(msd, orc, cuda, rows, cols, stable, half):
    _softmax_case(msd, orc, cuda, rows, cols, 8000 + cols, half, stable, inplace=True)


@pytest.mark.parametrize("rows,cols", [(1, 1), (3, 4), (5, 8), (9, 40), (7, 300), (4, 600), (6, 1000),
                                       (3, 2048), (5, 8192), (2, 10000), (33, 129), (2, 513),
                                       (200, 100), (128, 9), (64, 128), (191, 127), (70, 8),
                                       # rows of 3 ... 66 vectors: every team size of the register kernel,
                                       # row counts that leave part of the last wavefront without a row
                                       (67, 24), (35, 32), (50, 96), (45, 200), (21, 136), (19, 264)])
def test_softmax_edge_shapes(msd, orc, cuda, rows, cols):
    for half in (False, True):
        for stable in (0, 1):
            _softmax_case(msd, orc, cuda, rows, cols, 8100 + cols, half, stable, sigma=1.5)


@pytest.mark.parametrize("rb", [16, 32, 64])
def test_softmax_short_rows_flat_kernel(msd, orc, cuda, rb):
    """Rows of 77 / 100 moved as flat 16-byte vectors, rb rows per workgroup, plus a ragged tail."""
    lib = msd.load_library()
    assert lib.msd_set_tuning(msd.TUNE_SOFTMAX_ROWS, rb) == 0
    try:
        for rows, cols in [(rb * 5 + 3, 77), (rb, 100), (2 * rb + 1, 9), (rb * 3, 127)]:
            for half in (False, True):
                for stable in (0, 1):
                    _softmax_case(msd, orc, cuda, rows, cols, 8300 + cols + rb, half, stable, inplace=True)
    finally:
        assert lib.msd_set_tuning(msd.TUNE_SOFTMAX_ROWS, 0) == 0
    assert lib.msd_set_tuning(msd.TUNE_SOFTMAX_ROWS, 48) == 1


@pytest.mark.parametrize("rows,cols,half,knob", [
    (12288 + 7, 77, True, 0), (20000, 100, False, 0),    # 16 lanes per row, 32 / 16 rows per workgroup
    (40000 + 3, 77, False, 0), (40000, 100, True, 0),    # 8 lanes per row, 64 / 32 rows
    (66000 + 1, 77, True, 0), (66000, 100, True, 0),     # 4 lanes per row up to 80 columns, 8 beyond
    (66000, 77, False, 16), (66000, 33, True, 32), (40000, 127, True, 16), (40000, 9, False, 64)])
def test_softmax_flat_kernel_lanes_per_row(msd, orc, cuda, rows, cols, half, knob):
    """Row counts on both sides of the limits where the flat kernel changes its lanes per row."""
    lib = msd.load_library()
    assert lib.msd_set_tuning(msd.TUNE_SOFTMAX_ROWS, knob) == 0
    try:
        for stable in (0, 1):
            _softmax_case(msd, orc, cuda, rows, cols, 8500 + cols + stable, half, stable, inplace=bool(stable))
    finally:
        assert lib.msd_set_tuning(msd.TUNE_SOFTMAX_ROWS, 0) == 0


def test_softmax_cross_attention_full_rows(msd, orc, cuda):
    """All 2 x 8 x 4096 query rows against 77 text tokens (the size that takes the flat kernel)."""
    _softmax_case(msd, orc, cuda, 2 * 8 * 4096, 77, 8400, True, 0, inplace=True)
    _softmax_case(msd, orc, cuda, 2 * 8 * 4096 + 5, 77, 8401, False, 1)


def test_softmax_overflow_follows_the_reference_unless_stable(msd, orc, cuda):
    x = np.zeros((2, 64), dtype=np.float32)
    x[0, 1], x[0, 2] = 89.0, 1.0
    x[1, :] = np.linspace(-3, 3, 64)
    with np.errstate(all="ignore"):
        ref = orc.softmax(x)
    got = msd.softmax(_to_dev(x, cuda), stable=False).cpu().numpy()
    assert np.isnan(ref[0, 1]) and np.isnan(got[0, 1])
    assert got[0, 0] == 0.0 and got[0, 2] == 0.0
    assert_close_f32(got[1], ref[1], what="finite row next to an overflowing one")
    safe = msd.softmax(_to_dev(x, cuda), stable=True).cpu().numpy()
    np.testing.assert_allclose(safe, orc.softmax64(x), rtol=1e-5, atol=1e-30)


def test_softmax_full_size_rows_sum_to_one(msd, cuda):
    """One attention map of the first UNet level at full size: 8 heads x 4096 x 4096, fp16, in place."""
    torch = _torch()
    g = torch.Generator(device=cuda)
    g.manual_seed(8200)
    x = torch.randn((8 * 4096, 4096), device=cuda, dtype=torch.float16, generator=g) * 3.0
    keep = x[:64].float().cpu().numpy()
    msd.softmax(x, stable=False, out=x)
    sums = x.float().sum(dim=-1)
    assert float((sums - 1.0).abs().max()) < 2e-2  # 4096 values rounded to fp16 each
    assert float(x.min()) >= 0.0 and float(x.max()) <= 1.0
    e = np.exp(keep.astype(np.float64))
    assert_close_f16(x[:64].float().cpu().numpy(), e / e.sum(axis=-1, keepdims=True), "softmax 65536x4096, 64 rows",
                     rel_floor=0.0)


# ----------------------------------------------------------------- DDIM
def test_ddim_schedule_is_bit_exact(msd, orc):
    assert np.array_equal(np.asarray(msd.alphas_cumprod(), dtype=np.float32), orc.alphas_cumprod())
    for steps in (50, 25, 30, 7, 1, 500):
        got, ref = msd.ddim_schedule(steps), orc.ddim_schedule(steps)
        for g, r in zip(got, ref):
            assert np.array_equal(np.asarray(g, dtype=r.dtype), r)
    lib = msd.load_library()
    assert lib.msd_ddim_schedule(0, None, None, None, None, 0) == -1
    assert lib.msd_ddim_schedule(501, None, None, None, None, 0) == -2


@pytest.mark.parametrize("n", [4 * 64 * 64, 2 * 4 * 64 * 64, 1001, 3, 1])
def test_ddim_update_fp32_is_bit_exact(msd, orc, cuda, n):
    x = orc.normal((n,), seed=9000 + n)
    e = orc.normal((n,), seed=9100 + n)
    ts, a, ap, s1m = orc.ddim_schedule(50)
    for index in (49, 30, 0):
        ref = orc.ddim_update(x, e, a[index], ap[index], s1m[index])
        xd = _to_dev(x, cuda)
        got = msd.ddim_update(xd, _to_dev(e, cuda), float(a[index]), float(ap[index]), float(s1m[index]))
        assert np.array_equal(got.cpu().numpy(), ref)
        msd.ddim_update(xd, _to_dev(e, cuda), float(a[index]), float(ap[index]), float(s1m[index]), out=xd)
        assert np.array_equal(xd.cpu().numpy(), ref)


def test_ddim_update_fixture_unaligned_and_fp16(msd, orc, cuda, golden):
    x, e = golden["ddim_x"], golden["ddim_e"]
    a_t, a_prev = np.float32(golden["ddim_a_t"]), np.float32(golden["ddim_a_prev"])
    s1m = np.sqrt(np.float32(1.0) - a_t)
    got = msd.ddim_update(_to_dev(x, cuda), _to_dev(e, cuda), float(a_t), float(a_prev), float(s1m))
    assert_close_f32(got.cpu().numpy(), golden["ddim_x_prev_f64"], 2e-6, "ddim vs LDM f64")
    xo = _to_dev(np.concatenate([[0.0], x]).astype(np.float32), cuda)[1:]
    eo = _to_dev(np.concatenate([[0.0], e]).astype(np.float32), cuda)[1:]
    got = msd.ddim_update(xo, eo, float(a_t), float(a_prev), float(s1m))
    assert np.array_equal(got.cpu().numpy(), orc.ddim_update(x, e, a_t, a_prev, s1m))
    xh, eh = orc.round_to_half(x), orc.round_to_half(e)
    goth = msd.ddim_update(_to_dev(xh, cuda, True), _to_dev(eh, cuda, True), float(a_t), float(a_prev), float(s1m))
    ref16 = orc.round_to_half(orc.ddim_update(xh, eh, a_t, a_prev, s1m))
    assert np.array_equal(goth.float().cpu().numpy(), ref16)  # same float32 value, rounded once


def test_ddim_sampling_loop_is_bit_exact(msd, orc, cuda):
    """25 steps, walked from the back as the sampler does, with a stand-in noise model."""
    ts, a, ap, s1m = orc.ddim_schedule(25)
    x = orc.normal((4 * 64 * 64,), seed=9201)
    noise = orc.normal((4 * 64 * 64,), seed=9202)
    xd, nd = _to_dev(x, cuda), _to_dev(noise, cuda)
    for index in range(len(ts) - 1, -1, -1):
        scale = np.float32(0.25 + 0.001 * ts[index])
        e = (np.float32(0.5) * x + scale * noise).astype(np.float32)
        ed = xd * 0.5 + nd * float(scale)  # torch float32 elementwise: same roundings as numpy
        x = orc.ddim_update(x, e, a[index], ap[index], s1m[index])
        msd.ddim_update(xd, ed, float(a[index]), float(ap[index]), float(s1m[index]), out=xd)
    assert np.array_equal(xd.cpu().numpy(), x)
