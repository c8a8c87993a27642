"""Parity of the HIP kernels (through the C ABI) against the CPU oracle.

Same seeded inputs go to the oracle (float32 restatement of the reference's
kernels) and to the GPU.  fp32 storage: 1e-5 relative; fp16 storage: the oracle
runs on fp16-rounded inputs and the stored fp16 result must be the correct
rounding of a value within 1e-5 of its unrounded output (see tolerances.py).  Shapes are the reference's SD UNet / text-encoder shapes at
batch 2 plus the edge cases the reference's preconditions and the kernels'
dispatch split on.
"""
import numpy as np
import pytest

from tolerances import assert_close_f16, assert_close_f32

pytestmark = pytest.mark.gpu

# (channels, height*width) of every GroupNorm in one UNet step; in-norm and out-norm
# of the 22 ResBlocks (M/UNetModel.cpp:86-1018) and the final norm (:1007)
UNET_GN_SHAPES = sorted({
    (320, 4096), (640, 4096), (960, 4096), (320, 1024), (640, 1024), (1280, 1024), (960, 1024),
    (1920, 1024), (640, 256), (1280, 256), (1920, 256), (2560, 256), (1280, 64), (2560, 64),
})
CFG2_SHAPES = [(320, 4096, 2001), (640, 1024, 2002), (1280, 256, 2003), (1280, 64, 2004),
               (960, 1024, 2005), (1920, 256, 2006)]


def _torch():
    import torch
    return torch


def _to_dev(a, cuda, half=False):
    torch = _torch()
    t = torch.from_numpy(np.ascontiguousarray(a)).to(cuda)
    return t.half() if half else t


def _affine(orc, channels, seed):
    return (orc.normal((channels,), seed=seed + 500000, mean=1.0, sigma=0.1),
            orc.normal((channels,), seed=seed + 600000, mean=0.0, sigma=0.1))


def _run_groupnorm(msd, orc, cuda, x, g, b, groups, eps, silu, half, inplace=False):
    xin = orc.round_to_half(x) if half else x
    ref = orc.groupnorm(xin, g, b, groups, eps, silu)
    xd = _to_dev(xin, cuda, half)
    out = msd.groupnorm(xd, _to_dev(g, cuda), _to_dev(b, cuda), groups, eps, silu,
                        out=xd if inplace else None)
    got = out.float().cpu().numpy()
    if half:
        return assert_close_f16(got, ref, "groupnorm f16 %s" % (x.shape,))
    return assert_close_f32(got, ref, what="groupnorm f32 %s" % (x.shape,)), None


# ----------------------------------------------------------------- GroupNorm
@pytest.fixture(params=[0, 1], ids=["writers-auto", "one-writer"])
def gn_writers(request, msd):
    """Runs a test twice: with the launch plan free to let several workgroups share a whole
    (sample, group) when the output lies apart from the input, and with that switched off (one
    workgroup per unit or slices with an exchange, as for a call in place)."""
    lib = msd.load_library()
    assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, request.param) == 0
    yield request.param
    assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, 0) == 0


def test_config1_groupnorm_silu_fp32(msd, orc, cuda, gn_writers):
    x = orc.normal((1, 320, 64, 64), seed=1001)
    g, b = _affine(orc, 320, 1001)
    _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, half=False)
    assert msd.status() == 0


@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
@pytest.mark.parametrize("channels,hw,seed", CFG2_SHAPES)
def test_config2_groupnorm_silu_sweep(msd, orc, cuda, channels, hw, seed, half, gn_writers):
    side = int(round(hw ** 0.5))
    x = orc.normal((2, channels, side, side), seed=seed, sigma=2.0)
    g, b = _affine(orc, channels, seed)
    worst, exact = _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, half)
    if half:
        assert exact > 0.99  # nearly every element is bit-identical to the rounded oracle
    assert msd.status() == 0


@pytest.mark.parametrize("channels,hw", UNET_GN_SHAPES)
def test_unet_step_groupnorm_shapes_fp16(msd, orc, cuda, channels, hw, gn_writers):
    x = orc.normal((2, channels, hw), seed=5001 + channels + hw, sigma=1.5, mean=0.2)
    g, b = _affine(orc, channels, 5001 + channels)
    _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, half=True)


@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
def test_groupnorm_in_place_and_no_silu(msd, orc, cuda, half, gn_writers):
    # in place as at M/nn/ResBlock.cpp:222; eps 1e-6 without SiLU as in SpatialTransformer
    x = orc.normal((2, 640, 32, 32), seed=77, sigma=1.0, mean=-0.5)
    g, b = _affine(orc, 640, 77)
    _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, half, inplace=True)
    _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-6, False, half, inplace=True)
    _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-6, False, half)


@pytest.mark.parametrize("split,threads", [(1, 0), (2, 0), (4, 0), (8, 256), (16, 0), (64, 64), (2, 1024),
                                           (4, 320), (1, 640)])
def test_groupnorm_every_split_factor(msd, orc, cuda, split, threads):
    # the same tensor through 1 .. 64 workgroups per group must agree with the oracle
    lib = msd.load_library()
    x = orc.normal((2, 320, 64, 64), seed=88, sigma=2.0, mean=1.0)
    g, b = _affine(orc, 320, 88)
    try:
        assert lib.msd_set_tuning(msd.TUNE_GN_SPLIT, split) == 0
        assert lib.msd_set_tuning(msd.TUNE_GN_THREADS, threads) == 0
        for half in (False, True):
            _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, half)
            _run_groupnorm(msd, orc, cuda, x[:1, :96, :24, :24].copy(), g[:96], b[:96], 32, 1e-5, True, half)
    finally:
        lib.msd_set_tuning(msd.TUNE_GN_SPLIT, 0)
        lib.msd_set_tuning(msd.TUNE_GN_THREADS, 0)
    assert msd.status() == 0


@pytest.mark.parametrize("threads", [256, 320, 384, 448, 512, 576, 640, 768])
def test_groupnorm_many_vectors_per_lane(msd, orc, cuda, threads):
    """Small workgroups that hold 8 - 20 vectors per lane (what large batches run): exact and
    ragged fits, gamma / beta through LDS, with and without SiLU, in place, with the ResBlock's
    embedding add folded in, and one unit cut in two."""
    import torch
    lib = msd.load_library()
    x = orc.normal((3, 320, 64, 64), seed=311 + threads, sigma=1.5, mean=0.4)
    g, b = _affine(orc, 320, 311)
    emb = orc.normal((3, 320), seed=312, sigma=0.5)
    try:
        assert lib.msd_set_tuning(msd.TUNE_GN_THREADS, threads) == 0
        for half in (True, False):
            _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, half)
            _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-6, False, half, inplace=True)
            # a ragged fit: 9 channels of 64 x 48 per group
            _run_groupnorm(msd, orc, cuda, x[:2, :288, :, :48].copy(), g[:288], b[:288], 32, 1e-5, True, half)
            # chunkwise_add + GroupNorm in one launch against the two passes of the oracle
            xin = orc.round_to_half(x) if half else x
            ein = orc.round_to_half(emb) if half else emb
            summed = xin + ein[:, :, None, None]
            summed = orc.round_to_half(summed) if half else summed.astype(np.float32)
            ref = orc.groupnorm(summed, g, b, 32, 1e-5, True)
            got = msd.chunk_add_groupnorm(_to_dev(xin, cuda, half), _to_dev(ein, cuda, half), _to_dev(g, cuda),
                                          _to_dev(b, cuda), 32, 1e-5, True).float().cpu().numpy()
            if half:
                assert_close_f16(got, ref, "chunk add groupnorm, %d lanes" % threads)
            else:
                assert_close_f32(got, ref, what="chunk add groupnorm f32, %d lanes" % threads)
        assert lib.msd_set_tuning(msd.TUNE_GN_SPLIT, 2) == 0
        _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, True)
        _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, False)
    finally:
        lib.msd_set_tuning(msd.TUNE_GN_THREADS, 0)
        lib.msd_set_tuning(msd.TUNE_GN_SPLIT, 0)
    assert msd.status() == 0


@pytest.mark.parametrize("batch,channels,hw,half", [
    (3, 320, 4096, True), (3, 960, 4096, True), (5, 320, 4096, True), (6, 640, 4096, True), (5, 960, 1024, False),
    (6, 1920, 1024, False), (7, 640, 1024, False), (10, 640, 4096, True), (12, 640, 4096, True), (10, 320, 4096, False),
    (16, 640, 1024, True)])
def test_groupnorm_plans_at_the_batches_in_between(msd, orc, cuda, batch, channels, hw, half):
    """The launches the planning rule makes by itself between one and two workgroups per CU (no
    measured plan exists for these batches), in place as the reference's out-norms run and out of
    place."""
    code = msd.DTYPE_F16 if half else msd.DTYPE_F32
    assert msd.groupnorm_plan(batch, channels, hw, 32, code, False, True)[0] >= 1   # the register kernel
    x = orc.normal((batch, channels, hw), seed=batch * 1000 + channels, sigma=1.3, mean=0.4)
    g, b = _affine(orc, channels, batch + channels)
    _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, half, inplace=True)
    _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, half)
    assert msd.status() == 0


def test_groupnorm_large_batch_plan_and_wide_groups(msd, orc, cuda):
    """What the launch plan picks by itself for many units (batch 25: 800 units, 256 lanes x 20
    vectors; batch 17: 544 units, short units on 512 lanes), and a group of more channels than the
    LDS copy of gamma / beta holds (the general kernel takes over)."""
    lib = msd.load_library()
    x = orc.normal((25, 320, 64, 64), seed=521, sigma=1.2, mean=-0.3)
    g, b = _affine(orc, 320, 521)
    assert msd.groupnorm_plan(25, 320, 4096) == (1, 256, 20, 1)
    _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, True)
    _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, False)
    # the other unit sizes of the UNet at that batch: 10 and 5 vectors per lane, ragged 16 and 8
    for batch, channels, hw, plan in ((25, 640, 1024, (1, 256, 10, 1)), (25, 1280, 256, (1, 256, 5, 1)),
                                      (25, 960, 1024, (1, 256, 16, 1)), (25, 1920, 256, (1, 256, 8, 1)),
                                      (17, 640, 1024, (1, 512, 5, 1)), (17, 960, 1024, (1, 512, 8, 1))):
        assert msd.groupnorm_plan(batch, channels, hw) == plan
        xs = orc.normal((batch, channels, hw), seed=523 + channels, sigma=1.4, mean=0.2)
        gs, bs = _affine(orc, channels, 523 + channels)
        _run_groupnorm(msd, orc, cuda, xs, gs, bs, 32, 1e-5, True, True)
    wide = orc.normal((1, 32 * 1100, 16), seed=522, sigma=1.0)
    gw, bw = _affine(orc, 32 * 1100, 522)
    try:
        assert lib.msd_set_tuning(msd.TUNE_GN_THREADS, 256) == 0  # 2200 vectors on 256 lanes: 10 per lane
        _run_groupnorm(msd, orc, cuda, wide, gw, bw, 32, 1e-5, True, True)
    finally:
        lib.msd_set_tuning(msd.TUNE_GN_THREADS, 0)
    assert msd.status() == 0


@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
def test_groupnorm_and_layernorm_non_finite_inputs_poison_their_unit_only(msd, orc, cuda, half):
    """An infinity or a NaN in the input makes the statistics of its (sample, group) / row NaN in
    the reference's arithmetic (K/group_norm.cl:1-76, K/layer_norm.cl:1-78: inf - inf), so that unit
    comes out all NaN and every other unit is untouched; the same must hold here, for whole units
    and for units cut in slices (the slices exchange the NaN)."""
    x = orc.normal((2, 320, 64, 64), seed=641, sigma=1.0)
    x[0, 5, 3, 7] = np.inf          # group 0 of sample 0
    x[1, 315, 60, 1] = np.nan       # group 31 of sample 1
    x[1, 100, 0, 0] = -np.inf       # group 10 of sample 1
    g, b = _affine(orc, 320, 641)
    xin = orc.round_to_half(x) if half else x
    for shape in ((2, 320, 64, 64), (2, 320, 16, 16)):
        xs = np.ascontiguousarray(xin[:, :, :shape[2], :shape[3]])
        ref = orc.groupnorm(xs, g, b, 32, 1e-5, True)
        got = msd.groupnorm(_to_dev(xs, cuda, half), _to_dev(g, cuda), _to_dev(b, cuda), 32, 1e-5, True).float().cpu().numpy()
        assert np.array_equal(np.isnan(got), np.isnan(ref))
        bad = np.isnan(ref).reshape(2, 32, -1)
        poisoned = (~np.isfinite(xs)).reshape(2, 32, -1).any(axis=2)
        assert poisoned.sum() >= 2
        assert np.array_equal(bad.all(axis=2), poisoned) and np.array_equal(bad.any(axis=2), poisoned)
        ok = ~np.isnan(ref)
        if half:
            assert_close_f16(got[ok], ref[ok], "groupnorm f16 with non-finite units")
        else:
            assert_close_f32(got[ok], ref[ok], what="groupnorm f32 with non-finite units")
    rows = xin.reshape(-1, 320)[:4096].copy()
    rows[7, 300] = np.inf
    rows[4000, 0] = np.nan
    ref = orc.layernorm(rows, g, b, 1e-5)
    got = msd.layernorm(_to_dev(rows, cuda, half), _to_dev(g, cuda), _to_dev(b, cuda), 1e-5).float().cpu().numpy()
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    ok = ~np.isnan(ref)
    assert np.isnan(ref).all(axis=1).sum() >= 2
    if half:
        assert_close_f16(got[ok], ref[ok], "layernorm f16 with non-finite rows")
    else:
        assert_close_f32(got[ok], ref[ok], what="layernorm f32 with non-finite rows")
    assert msd.status() == 0


@pytest.mark.parametrize("split", [2, 4, 16])
def test_groupnorm_slice_that_stops_waiting_computes_its_siblings_statistics(msd, orc, cuda, split):
    """With a poll limit of one, nearly every workgroup gives up on its siblings at once and
    computes their statistics from the input itself (what a starved workgroup does after a
    millisecond in normal operation).  Every kernel still runs to its normal end and the
    output must be the usual one, in place too (siblings overwrite their part of the input only
    after they have seen every word of the unit)."""
    lib = msd.load_library()
    x = orc.normal((2, 320, 64, 64), seed=97, sigma=2.0, mean=1.0)
    g, b = _affine(orc, 320, 97)
    msd.gn_fallbacks(reset=True)
    try:
        assert lib.msd_set_tuning(msd.TUNE_GN_SPLIT, split) == 0
        assert lib.msd_set_tuning(msd.TUNE_GN_SPIN_LIMIT, 1) == 0
        for half in (False, True):
            for inplace in (False, True):
                _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, half, inplace=inplace)
        # the token-major kernel shares the exchange
        xin = orc.round_to_half(x[:, :, :32, :32])
        tok = msd.groupnorm_tokens(_to_dev(xin, cuda, True), _to_dev(g, cuda), _to_dev(b, cuda), 32, 1e-6)
        ref = orc.groupnorm(xin, g, b, 32, 1e-6, False).reshape(2, 320, -1).transpose(0, 2, 1)
        assert_close_f16(tok.float().cpu().numpy(), ref, "gn tokens, forced give-up")
    finally:
        lib.msd_set_tuning(msd.TUNE_GN_SPLIT, 0)
        lib.msd_set_tuning(msd.TUNE_GN_SPIN_LIMIT, 0)
    assert msd.gn_fallbacks() > 0  # the path was really taken
    # back to the normal limit: no workgroup gives up on an idle GPU
    msd.gn_fallbacks(reset=True)
    _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, True, inplace=True)
    assert msd.gn_fallbacks() == 0
    assert msd.status() == 0


def test_groupnorm_repeated_launches_reuse_scratch(msd, orc, cuda):
    # the arrival counters are never reset: many launches with changing split factors
    lib = msd.load_library()
    shapes = [(2, 320, 4096), (2, 1280, 64), (1, 640, 1024), (2, 1920, 256), (2, 320, 4096)]
    try:
        for rep in range(3):
            for i, shp in enumerate(shapes):
                lib.msd_set_tuning(msd.TUNE_GN_SPLIT, [4, 2, 8, 1][(rep + i) % 4])
                x = orc.normal(shp, seed=900 + i + 10 * rep, sigma=2.0)
                g, b = _affine(orc, shp[1], 900 + i)
                _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, half=True)
    finally:
        lib.msd_set_tuning(msd.TUNE_GN_SPLIT, 0)
    assert msd.status() == 0


@pytest.mark.parametrize("shape,groups", [
    ((1, 32, 3, 3), 32),      # hw not a multiple of the vector width: scalar kernel
    ((3, 64, 5, 7), 8),       # odd everything
    ((2, 64, 2, 4), 32),      # one 16-byte vector per channel (fp16)
    ((1, 96, 24, 24), 32),    # ragged slices: 3 channels per group
    ((5, 32, 40, 40), 4),     # few large groups, odd batch
    ((1, 4, 512, 512), 1),    # one huge group: maximum split
])
@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
def test_groupnorm_edge_shapes(msd, orc, cuda, shape, groups, half, gn_writers):
    x = orc.normal(shape, seed=sum(shape), sigma=1.3, mean=0.1)
    xin = orc.round_to_half(x) if half else x
    g, b = _affine(orc, shape[1], 31)
    ref = orc.groupnorm64(xin, g, b, groups, 1e-5, True)  # textbook: these shapes break the
    xd = _to_dev(xin, cuda, half)                         # reference's % 64 precondition
    got = msd.groupnorm(xd, _to_dev(g, cuda), _to_dev(b, cuda), groups, 1e-5, True).float().cpu().numpy()
    if half:
        assert_close_f16(got, ref.astype(np.float32), "gn edge f16")
    else:
        assert_close_f32(got, ref, what="gn edge f32")
    assert msd.status() == 0


def test_groupnorm_misaligned_and_empty(msd, orc, cuda):
    torch = _torch()
    x = orc.normal((1, 64, 8, 8), seed=5)
    g, b = _affine(orc, 64, 5)
    ref = orc.groupnorm(x, g, b, 32, 1e-5, True)
    buf = torch.zeros(x.size + 1, device=cuda)
    buf[1:] = torch.from_numpy(x.reshape(-1)).to(cuda)
    xin = buf[1:].view(1, 64, 8, 8)  # 4-byte aligned only
    got = msd.groupnorm(xin, _to_dev(g, cuda), _to_dev(b, cuda), 32, 1e-5, True).cpu().numpy()
    assert_close_f32(got, ref, what="gn misaligned")
    empty = torch.empty((0, 64, 8, 8), device=cuda)
    assert msd.groupnorm(empty, _to_dev(g, cuda), _to_dev(b, cuda), 32).numel() == 0
    lib = msd.load_library()
    assert lib.msd_groupnorm(None, None, None, None, 1, 30, 16, 32, 1e-5, 0, 0, None) == 1
    assert lib.msd_groupnorm(None, None, None, None, 1, 32, 16, 32, 1e-5, 0, 7, None) == 1


def test_groupnorm_statistics_property_full_size(msd, orc, cuda):
    # size-independent check at the largest UNet shape: unit statistics per (sample, group)
    torch = _torch()
    x = torch.randn((2, 960, 64, 64), device=cuda, generator=torch.Generator(device=cuda).manual_seed(3)) * 3 + 1
    one, zero = torch.ones(960, device=cuda), torch.zeros(960, device=cuda)
    y = msd.groupnorm(x, one, zero, 32, 1e-5, False).double().view(2, 32, -1)
    assert y.mean(dim=2).abs().max().item() < 1e-5
    assert (y.var(dim=2, unbiased=False) - 1.0).abs().max().item() < 1e-4
    # affine linearity: GN(x; g, b) == g * GN(x; 1, 0) + b
    g = torch.rand(960, device=cuda) + 0.5
    b = torch.randn(960, device=cuda)
    y2 = msd.groupnorm(x, g, b, 32, 1e-5, False)
    base = msd.groupnorm(x, one, zero, 32, 1e-5, False)
    assert (y2 - (base * g.view(1, -1, 1, 1) + b.view(1, -1, 1, 1))).abs().max().item() < 1e-5
    assert msd.status() == 0


@pytest.mark.parametrize("mean,sigma", [(5.0, 1.0), (50.0, 1.0), (500.0, 1.0), (1.0, 0.01), (100.0, 0.01),
                                        (1e4, 10.0), (0.0, 1e-4)])
def test_groupnorm_ill_conditioned_inputs_track_float64_like_the_reference(msd, orc, cuda, mean, sigma, gn_writers):
    """With |mean| >> sigma float32 itself cannot hold 1e-5 (the reference's two-pass algorithm is
    1e-4 .. 1e-3 away from float64 there).  The kernel must then be no further from float64
    than that restatement is (it is closer: centred statistics per wavefront, Chan merges)."""
    x = orc.normal((2, 320, 64, 64), seed=3, mean=mean, sigma=sigma)
    g, b = np.ones(320, np.float32), np.zeros(320, np.float32)
    ref64 = orc.groupnorm64(x, g, b, 32, 1e-5, False)
    ref32 = orc.groupnorm(x, g, b, 32, 1e-5, False)
    got = msd.groupnorm(_to_dev(x, cuda), _to_dev(g, cuda), _to_dev(b, cuda), 32, 1e-5, False).cpu().numpy()

    def err(a):
        return float(np.max(np.abs(a.astype(np.float64) - ref64) / np.maximum(1.0, np.abs(ref64))))
    assert err(got) <= 1.25 * err(ref32) + 1e-6


def test_groupnorm_golden_fixtures(msd, golden, cuda):
    for name in ("gn_a", "gn_b", "gn_c"):
        x, g, b = (_to_dev(golden[name + k], cuda) for k in ("_x", "_gamma", "_beta"))
        eps = float(golden[name + "_eps"])
        assert_close_f32(msd.groupnorm(x, g, b, 32, eps, False).cpu().numpy(), golden[name + "_y"], what=name)
        assert_close_f32(msd.groupnorm(x, g, b, 32, eps, True).cpu().numpy(), golden[name + "_y_silu"], what=name)


# ----------------------------------------------------------------- LayerNorm
@pytest.mark.parametrize("rows,dim,seed", [(8192, 320, 3001), (2048, 640, 3002), (512, 1280, 3003),
                                           (128, 1280, 3007)])
def test_config3_layernorm_fp16(msd, orc, cuda, rows, dim, seed):
    x = orc.round_to_half(orc.normal((2, rows // 2, dim), seed=seed))
    g, b = _affine(orc, dim, seed)
    ref = orc.layernorm(x, g, b, 1e-5)
    got = msd.layernorm(_to_dev(x, cuda, True), _to_dev(g, cuda), _to_dev(b, cuda)).float().cpu().numpy()
    worst, exact = assert_close_f16(got, ref, "layernorm f16 %dx%d" % (rows, dim))
    assert exact > 0.99


@pytest.mark.parametrize("rows,dim,seed", [(77, 768, 4001), (154, 768, 4002), (77, 1024, 4004)])
def test_config4_layernorm_fp32_outliers(msd, orc, cuda, rows, dim, seed):
    x = orc.add_outliers(orc.normal((rows, dim), seed=seed), seed=seed)
    g, b = _affine(orc, dim, seed)
    got = msd.layernorm(_to_dev(x, cuda), _to_dev(g, cuda), _to_dev(b, cuda)).cpu().numpy()
    assert_close_f32(got, orc.layernorm(x, g, b, 1e-5), what="layernorm f32 outliers")


@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
@pytest.mark.parametrize("rows,dim", [(1, 64), (3, 128), (5, 192), (9, 320), (33, 448), (7, 576),
                                      (4, 2048), (3, 4096), (2, 8192), (5, 100), (6, 36), (2, 7),
                                      (3, 6400)])
def test_layernorm_dims_and_ragged_rows(msd, orc, cuda, rows, dim, half):
    # every team width / vectors-per-lane pairing, the scalar kernel (dim 100, 36, 7) and
    # row counts that do not fill the last wavefront
    x = orc.normal((rows, dim), seed=rows * 1000 + dim, sigma=2.0, mean=3.0)
    xin = orc.round_to_half(x) if half else x
    g, b = _affine(orc, dim, dim)
    ref = orc.layernorm64(xin, g, b, 1e-5)
    got = msd.layernorm(_to_dev(xin, cuda, half), _to_dev(g, cuda), _to_dev(b, cuda)).float().cpu().numpy()
    if half:
        assert_close_f16(got, ref.astype(np.float32), "ln dims f16")
    else:
        assert_close_f32(got, ref, what="ln dims f32")


@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
@pytest.mark.parametrize("rows,dim", [(2049, 1024), (5001, 1024), (10241, 768), (16387, 320), (9001, 640),
                                      (4097, 1280)])
def test_layernorm_mid_size_launches_with_ragged_ends(msd, orc, cuda, rows, dim, half):
    # launches of 2048 ... 10240 wavefronts: gamma / beta through LDS in workgroups of two or
    # four wavefronts, the last workgroup only partly filled with rows; alone and with the
    # residual added first
    x = orc.normal((rows, dim), seed=rows + dim, sigma=1.5, mean=0.5)
    r = orc.normal((rows, dim), seed=rows + dim + 1)
    if half:
        x, r = orc.round_to_half(x), orc.round_to_half(r)
    g, b = _affine(orc, dim, dim)
    gd, bd = _to_dev(g, cuda), _to_dev(b, cuda)
    check = (lambda got, ref, what: assert_close_f16(got, ref.astype(np.float32), what)) if half else \
            (lambda got, ref, what: assert_close_f32(got, ref, what=what))
    got = msd.layernorm(_to_dev(x, cuda, half), gd, bd).float().cpu().numpy()
    check(got, orc.layernorm64(x, g, b, 1e-5), "ln mid-size")
    s = x + r
    if half:
        s = orc.round_to_half(s)
    sm, got = msd.add_layernorm(_to_dev(x, cuda, half), _to_dev(r, cuda, half), gd, bd, 1e-5)
    assert np.array_equal(sm.float().cpu().numpy(), s.astype(np.float32))
    check(got.float().cpu().numpy(), orc.layernorm64(s.astype(np.float32), g, b, 1e-5), "add + ln mid-size")


@pytest.mark.parametrize("chunk,threads", [(8, 0), (16, 0), (8, 64), (16, 512), (0, 128)])
def test_layernorm_forced_chunk_width(msd, orc, cuda, chunk, threads):
    lib = msd.load_library()
    try:
        assert lib.msd_set_tuning(msd.TUNE_LN_CHUNK, chunk) == 0
        assert lib.msd_set_tuning(msd.TUNE_LN_THREADS, threads) == 0
        for rows, dim, half in [(8192, 320, True), (300, 640, True), (77, 768, False), (33, 1280, False),
                                (5, 64, True), (5, 64, False), (9, 2048, True)]:
            x = orc.normal((rows, dim), seed=rows + dim + chunk, sigma=1.5, mean=-1.0)
            xin = orc.round_to_half(x) if half else x
            g, b = _affine(orc, dim, dim + 1)
            ref = orc.layernorm(xin, g, b, 1e-5)
            got = msd.layernorm(_to_dev(xin, cuda, half), _to_dev(g, cuda), _to_dev(b, cuda)).float().cpu().numpy()
            if half:
                assert_close_f16(got, ref, "ln chunk f16")
            else:
                assert_close_f32(got, ref, what="ln chunk f32")
    finally:
        lib.msd_set_tuning(msd.TUNE_LN_CHUNK, 0)
        lib.msd_set_tuning(msd.TUNE_LN_THREADS, 0)


def test_layernorm_in_place_fixtures_and_empty(msd, orc, golden, cuda):
    torch = _torch()
    for name in ("ln_a", "ln_b", "ln_c", "ln_d"):
        x, g, b = (_to_dev(golden[name + k], cuda) for k in ("_x", "_gamma", "_beta"))
        y = msd.layernorm(x, g, b, float(golden[name + "_eps"]), out=x)  # in place
        assert_close_f32(y.cpu().numpy(), golden[name + "_y"], what=name)
    e = torch.empty((0, 320), device=cuda)
    assert msd.layernorm(e, torch.ones(320, device=cuda), torch.zeros(320, device=cuda)).numel() == 0


# ----------------------------------------------------------------- GEGLU and activations
@pytest.mark.parametrize("rows,inner,seed", [(8192, 1280, 3004), (2048, 2560, 3005), (512, 5120, 3006),
                                             (128, 5120, 3008)])
def test_config3_geglu_fp16(msd, orc, cuda, rows, inner, seed):
    proj = orc.round_to_half(orc.normal((rows, 2 * inner), seed=seed))
    ref = orc.geglu(proj)
    got = msd.geglu(_to_dev(proj, cuda, True)).float().cpu().numpy()
    worst, exact = assert_close_f16(got, ref, "geglu f16 %dx%d" % (rows, inner))
    assert exact > 0.99


@pytest.mark.parametrize("rows,inner", [(77, 1280), (5, 64), (3, 20), (7, 9), (1025, 8), (1, 1)])
@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
def test_geglu_shapes_fp32_fp16(msd, orc, golden, cuda, rows, inner, half):
    proj = orc.normal((rows, 2 * inner), seed=rows + inner, sigma=2.5)
    pin = orc.round_to_half(proj) if half else proj
    ref = orc.geglu(pin)
    got = msd.geglu(_to_dev(pin, cuda, half)).float().cpu().numpy()
    if half:
        assert_close_f16(got, ref, "geglu shapes f16")
    else:
        assert_close_f32(got, ref, what="geglu shapes f32")
        assert_close_f32(msd.geglu(_to_dev(golden["geglu_proj"], cuda)).cpu().numpy(), golden["geglu_y"])


@pytest.mark.parametrize("unroll", [1, 2, 4])
def test_geglu_forced_vectors_per_lane(msd, orc, cuda, unroll):
    lib = msd.load_library()
    try:
        assert lib.msd_set_tuning(msd.TUNE_GEGLU_VECTORS, unroll) == 0
        assert lib.msd_set_tuning(msd.TUNE_ACT_VECTORS, unroll) == 0
        x = orc.normal((3, 1031), seed=unroll, sigma=3.0)
        assert_close_f32(msd.silu(_to_dev(x, cuda)).cpu().numpy(), orc.silu(x), what="silu unroll")
        for rows, inner in [(2048, 2560), (77, 1288), (3, 8), (1000, 24)]:
            proj = orc.round_to_half(orc.normal((rows, 2 * inner), seed=rows + unroll, sigma=1.5))
            got = msd.geglu(_to_dev(proj, cuda, True)).float().cpu().numpy()
            assert_close_f16(got, orc.geglu(proj), "geglu unroll")
    finally:
        lib.msd_set_tuning(msd.TUNE_GEGLU_VECTORS, 0)
        lib.msd_set_tuning(msd.TUNE_ACT_VECTORS, 0)


@pytest.mark.parametrize("name", ["silu", "gelu", "quick_gelu"])
@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
def test_activations(msd, orc, golden, cuda, name, half):
    fn, ref_fn = getattr(msd, name), getattr(orc, name)
    cases = [orc.add_outliers(orc.normal((2, 77, 3072), seed=4003), seed=4003),  # config 4 MLP hidden, 1 % at +-20
             orc.add_outliers(orc.normal((77, 4096), seed=4005), seed=4005),  # the reference's size
             orc.normal((2, 1280), seed=5002),                   # SiLU on the time embedding
             golden["act_x"], orc.normal((1031,), seed=9, sigma=4.0), orc.normal((3,), seed=10)]
    for x in cases:
        xin = orc.round_to_half(x) if half else np.ascontiguousarray(x)
        xd = _to_dev(xin, cuda, half)
        got = fn(xd, out=xd).float().cpu().numpy()  # in place, like every reference call site
        if half:
            assert_close_f16(got, ref_fn(xin), name + " f16")
        else:
            assert_close_f32(got, ref_fn(xin), what=name + " f32")
    if not half:
        got = fn(_to_dev(golden["act_x"], cuda)).cpu().numpy()
        assert_close_f32(got, golden["act_" + name], what=name + " fixture")


def test_activations_on_every_finite_fp16_value(msd, orc, cuda):
    """All 63488 finite binary16 values through SiLU, GELU, quick_GELU and as the GEGLU gate,
    fp16 storage, against the oracle on the same values."""
    bits = np.arange(0x10000, dtype=np.uint32).astype(np.uint16)
    vals = bits.view(np.float16)
    x = vals[np.isfinite(vals)].astype(np.float32)
    assert x.size == 63488
    xd = _to_dev(x, cuda, True)
    for name in ("silu", "gelu", "quick_gelu"):
        got = getattr(msd, name)(xd).float().cpu().numpy()
        assert_close_f16(got, getattr(orc, name)(x), name + " every fp16 value")
    for value in (1.0, -0.75, 0.001):  # value half (first), gate half (second) = every fp16 value
        proj = np.concatenate([np.full_like(x, value), x])[None, :]
        got = msd.geglu(_to_dev(proj, cuda, True)).float().cpu().numpy()
        assert_close_f16(got, orc.geglu(orc.round_to_half(proj)), "geglu gate every fp16 value")
    # fp32 storage on the same points: the plain 1e-5 criterion
    xf = _to_dev(x, cuda)
    for name in ("silu", "gelu", "quick_gelu"):
        assert_close_f32(getattr(msd, name)(xf).cpu().numpy(), getattr(orc, name)(x), what=name + " fp16 grid, f32")


def test_activation_special_values(msd, cuda):
    torch = _torch()
    x = torch.tensor([0.0, -0.0, 100.0, -100.0, 1e-30, -1e-30, 88.0, -88.0, 30.0, -30.0], device=cuda)
    s = msd.silu(x).cpu().numpy()
    assert s[0] == 0 and s[2] == 100.0 and abs(s[3]) < 1e-30 and s[8] == 30.0
    ge = msd.gelu(x).cpu().numpy()
    assert ge[0] == 0 and ge[2] == 100.0 and abs(ge[3]) < 1e-30 and ge[6] == 88.0 and abs(ge[9]) < 1e-30
    assert np.isfinite(s).all() and np.isfinite(ge).all()
    # non-finite inputs behave like the reference's expression x * 0.5 * (1 + erf(x / sqrt 2))
    nf = msd.gelu(torch.tensor([float("inf"), float("nan")], device=cuda)).cpu().numpy()
    assert nf[0] == np.inf and np.isnan(nf[1])


# ----------------------------------------------------------------- timestep embedding + DDIM list
def test_timestep_embedding_all_timesteps(msd, orc, golden, cuda):
    torch = _torch()
    ts = np.arange(0, 1000, dtype=np.int64)
    got = msd.timestep_embedding(torch.from_numpy(ts).to(cuda), 320).cpu().numpy()
    ref = np.stack([orc.timestep_embedding(int(t)) for t in ts])
    assert_close_f32(got, ref, what="timestep embedding")
    assert (got == ref).mean() > 0.95  # same frequencies and angles; cos/sin differ by <= 1 ulp
    # t = 0 row is exactly [1.. | 0..]; column 0 is cos(t), sin(t)
    assert np.array_equal(got[0], np.concatenate([np.ones(160), np.zeros(160)]).astype(np.float32))
    k = golden["temb_t"]
    g2 = msd.timestep_embedding(torch.from_numpy(k).to(cuda), 320).cpu().numpy()
    assert np.abs(g2 - golden["temb_f64"]).max() < 1.3e-4  # |t| * ulp(freq) at t ~ 1000
    # fp16 storage and another dim / period
    h = msd.timestep_embedding(torch.from_numpy(ts[:64]).to(cuda), 320, dtype=torch.float16).float().cpu().numpy()
    assert_close_f16(h, ref[:64], "temb f16")
    o = msd.timestep_embedding(torch.tensor([13], device=cuda), 64, max_period=100.0).cpu().numpy()[0]
    assert_close_f32(o, orc.timestep_embedding(13, 64, 100.0))


def test_config5_timesteps_feed_embedding_bit_exact_integers(msd, orc, cuda):
    torch = _torch()
    for steps in (50, 25, 30, 1000, 1):
        assert msd.ddim_timesteps(steps) == orc.ddim_timesteps(steps)
    sched = msd.ddim_timesteps(25)[::-1]  # the sampler walks the list from the back
    assert sched[0] == 961 and sched[-1] == 1
    t = torch.tensor(sched, dtype=torch.int64, device=cuda)
    emb = msd.timestep_embedding(t, 320).cpu().numpy()
    ref = np.stack([orc.timestep_embedding(s) for s in sched])
    assert_close_f32(emb, ref)
    rnd = orc.uniform_int(2, 5001, 0, 999)
    emb2 = msd.timestep_embedding(torch.from_numpy(rnd).to(cuda), 320, dtype=torch.float16)
    assert emb2.shape == (2, 320)


# ----------------------------------------------------------------- launch machinery
def test_groupnorm_graph_replay_matches_eager(msd, orc, cuda):
    """The cross-workgroup exchange keeps per-unit launch counts in device memory, so a
    captured graph must give on every replay what the eager launch gives."""
    torch = _torch()
    stream = torch.cuda.Stream()
    shapes = [(2, 320, 4096), (2, 960, 1024), (2, 1280, 64), (2, 640, 4096)]
    xs0 = [orc.round_to_half(orc.normal(s, seed=700 + i, sigma=2.0)) for i, s in enumerate(shapes)]
    gbs = [_affine(orc, s[1], 700 + i) for i, s in enumerate(shapes)]
    with torch.cuda.stream(stream):
        msd.init()
        xs = [_to_dev(x, cuda, True) for x in xs0]
        ys = [torch.empty_like(x) for x in xs]
        zs = [x.clone() for x in xs]
        gd = [(_to_dev(g, cuda), _to_dev(b, cuda)) for g, b in gbs]

        def body():
            for x, y, z, (g, b) in zip(xs, ys, zs, gd):
                msd.groupnorm(x, g, b, 32, 1e-5, True, out=y)   # out of place
                msd.groupnorm(z, g, b, 32, 1e-6, False, out=z)  # in place
        body()
        torch.cuda.synchronize()
        eager = [(y.clone(), z.clone()) for y, z in zip(ys, zs)]
        for x, z in zip(xs, zs):
            z.copy_(x)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            body()
        for rep in range(5):
            for x, y, z in zip(xs, ys, zs):  # eager work between replays
                y.zero_()
                z.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            for y, z, (ey, ez) in zip(ys, zs, eager):
                assert torch.equal(y, ey) and torch.equal(z, ez), "replay %d differs from the eager result" % rep
        assert msd.status() == 0
    # and the eager result is the right one
    for x0, (g, b), (ey, ez) in zip(xs0, gbs, eager):
        assert_close_f16(ey.float().cpu().numpy(), orc.groupnorm(x0, g, b, 32, 1e-5, True), "gn graph")
        assert_close_f16(ez.float().cpu().numpy(), orc.groupnorm(x0, g, b, 32, 1e-6, False), "gn graph")


def test_groupnorm_two_streams_have_private_scratch(msd, orc, cuda):
    torch = _torch()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    x1 = orc.round_to_half(orc.normal((2, 640, 4096), seed=801, sigma=2.0))
    x2 = orc.round_to_half(orc.normal((2, 960, 4096), seed=802, sigma=1.0, mean=3.0))
    g1, b1 = _affine(orc, 640, 801)
    g2, b2 = _affine(orc, 960, 802)
    d1, d2 = _to_dev(x1, cuda, True), _to_dev(x2, cuda, True)
    a1 = (_to_dev(g1, cuda), _to_dev(b1, cuda))
    a2 = (_to_dev(g2, cuda), _to_dev(b2, cuda))
    torch.cuda.synchronize()
    outs1, outs2 = [], []
    for _ in range(20):  # interleaved submissions keep both streams busy at once
        with torch.cuda.stream(s1):
            outs1.append(msd.groupnorm(d1, *a1, 32, 1e-5, True))
        with torch.cuda.stream(s2):
            outs2.append(msd.groupnorm(d2, *a2, 32, 1e-5, True))
    torch.cuda.synchronize()
    r1 = orc.groupnorm(x1, g1, b1, 32, 1e-5, True)
    r2 = orc.groupnorm(x2, g2, b2, 32, 1e-5, True)
    for o in outs1:
        assert torch.equal(o, outs1[0])
    for o in outs2:
        assert torch.equal(o, outs2[0])
    assert_close_f16(outs1[0].float().cpu().numpy(), r1, "stream 1")
    assert_close_f16(outs2[0].float().cpu().numpy(), r2, "stream 2")
    lib = msd.load_library()
    import ctypes
    assert lib.msd_status(ctypes.c_void_p(s1.cuda_stream)) == 0
    assert lib.msd_status(ctypes.c_void_p(s2.cuda_stream)) == 0


def test_host_threads_on_streams_of_their_own_get_the_results_of_one_thread(msd, orc, cuda):
    """Four host threads, each with a stream of its own, call cut and whole GroupNorms (a first call
    per stream allocates that stream's scratch under the library's lock), LayerNorm and GEGLU at the
    same time; ctypes drops the interpreter lock for the length of each call.  Every thread must see
    the bits a single thread gets, and no launch error."""
    import ctypes
    import threading
    torch = _torch()
    lib = msd.load_library()
    x = orc.round_to_half(orc.normal((2, 640, 4096), seed=811, sigma=2.0, mean=0.5))      # units cut in slices
    xs = orc.round_to_half(orc.normal((2, 1280, 256), seed=812, sigma=1.0))               # whole units, several writers
    rows = orc.round_to_half(orc.normal((2048, 640), seed=813))
    proj = orc.round_to_half(orc.normal((512, 2 * 1280), seed=814))
    g, b = _affine(orc, 640, 811)
    gs, bs = _affine(orc, 1280, 812)
    gl, bl = _affine(orc, 640, 813)
    dev = [_to_dev(x, cuda, True), _to_dev(xs, cuda, True), _to_dev(rows, cuda, True), _to_dev(proj, cuda, True)]
    aff = [_to_dev(v, cuda) for v in (g, b, gs, bs, gl, bl)]
    torch.cuda.synchronize()

    def work():
        out = [msd.groupnorm(dev[0], aff[0], aff[1], 32, 1e-5, True),
               msd.groupnorm(dev[1], aff[2], aff[3], 32, 1e-6, False),
               msd.layernorm(dev[2], aff[4], aff[5], 1e-5),
               msd.geglu(dev[3])]
        inplace = dev[0].clone()
        msd.groupnorm(inplace, aff[0], aff[1], 32, 1e-5, True, out=inplace)
        return out + [inplace]

    expect = work()
    torch.cuda.synchronize()
    results, errors = {}, []

    def thread(i):
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                got = None
                for _ in range(10):
                    got = work()
                stream.synchronize()
                results[i] = (got, lib.msd_status(ctypes.c_void_p(stream.cuda_stream)), msd.gn_fallbacks())
        except Exception as e:  # noqa: BLE001 - reported by the asserting thread
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=thread, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    torch.cuda.synchronize()
    assert not errors, errors
    assert sorted(results) == [0, 1, 2, 3]
    ref = orc.groupnorm(x, g, b, 32, 1e-5, True)
    for i, (got, status, gave_up) in results.items():
        assert status == 0, "thread %d" % i
        for k, (a, e) in enumerate(zip(got, expect)):
            if gave_up and k in (0, 4):
                # a slice that was kept waiting by the other threads' launches computed its sibling's
                # statistics itself, in another order of summation: right, but not the same bits
                assert_close_f16(a.float().cpu().numpy(), ref, "thread %d, result %d after %d give-ups" % (i, k, gave_up))
            else:
                assert torch.equal(a, e), "thread %d, result %d (msd_gn_fallbacks = %d)" % (i, k, gave_up)
    assert_close_f16(expect[4].float().cpu().numpy(), ref, "threads gn in place")
    assert_close_f16(expect[0].float().cpu().numpy(), ref, "threads gn")
    assert_close_f16(expect[2].float().cpu().numpy(), orc.layernorm(rows, gl, bl, 1e-5), "threads ln")


@pytest.mark.parametrize("batch,channels,hw", [(8, 320, 4096), (4, 640, 4096), (8, 960, 1024), (5, 320, 4096)])
def test_groupnorm_larger_batches_pick_other_splits(msd, orc, cuda, batch, channels, hw, gn_writers):
    # 128 / 256 units: the launch plan cuts units in two or not at all instead of in four
    x = orc.normal((batch, channels, hw), seed=batch * 1000 + channels, sigma=1.5, mean=0.2)
    g, b = _affine(orc, channels, 77)
    _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, half=True)
    _run_groupnorm(msd, orc, cuda, x[:, :, : hw // 4], g, b, 32, 1e-5, True, half=False)
    assert msd.status() == 0


@pytest.mark.parametrize("batch,channels,hw,plan", [
    (1, 320, 4096, (4, 640, 4, 1)), (1, 640, 1024, (4, 640, 2, 1)), (1, 960, 4096, (8, 960, 4, 1)),
    (2, 960, 4096, (8, 960, 4, 1)), (2, 320, 4096, (2, 1024, 5, 1)), (2, 1920, 256, (1, 960, 4, 1)),
    (2, 640, 256, (1, 640, 2, 1)), (4, 640, 4096, (4, 512, 10, 1)), (4, 1920, 1024, (4, 512, 8, 1)),
    (8, 320, 4096, (2, 512, 10, 1)), (8, 640, 4096, (2, 512, 20, 1))])
def test_groupnorm_fp32_plans_at_unet_shapes(msd, orc, cuda, batch, channels, hw, plan):
    """4-byte elements are cut more often and into exact fits of up to four vectors per lane (the
    plans of a call in place, which is how the tensor is run here)."""
    assert msd.groupnorm_plan(batch, channels, hw, 32, msd.DTYPE_F32, in_place=True) == plan
    x = orc.normal((batch, channels, hw), seed=batch * 1000 + channels + hw, sigma=2.0, mean=-0.1)
    g, b = _affine(orc, channels, 78)
    _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, half=False, inplace=True)
    assert msd.status() == 0


@pytest.mark.parametrize("writers", [2, 4, 8, 16])
def test_groupnorm_several_writers_per_unit_give_the_bits_of_one(msd, orc, cuda, writers):
    """Several workgroups per whole (sample, group), each loading and reducing all of it and storing
    one part: the statistics are computed as by a single workgroup, so the output must be the same
    bit for bit - for full and ragged units, either element size, with and without SiLU, with the
    embedding addend, for units in whole rows of 8 (writers 8 blocks apart) and not (adjacent) -
    and a call in place must not take that launch at all."""
    torch = _torch()
    lib = msd.load_library()
    cases = [((2, 320, 64, 64), 32), ((2, 640, 32, 32), 32), ((1, 96, 24, 24), 32), ((3, 24, 40, 40), 3),
             ((2, 1280, 8, 8), 32), ((1, 64, 56, 72), 8), ((5, 32, 40, 40), 4), ((2, 960, 32, 32), 32)]
    try:
        for shape, groups in cases:
            for half in (True, False):
                channels = shape[1]
                x = orc.normal(shape, seed=sum(shape) + writers, sigma=1.8, mean=0.4)
                xin = orc.round_to_half(x) if half else x
                g, b = _affine(orc, channels, 83)
                emb = orc.normal((shape[0], channels), seed=84, sigma=0.5)
                emb = orc.round_to_half(emb) if half else emb
                xd, gd, bd, ed = _to_dev(xin, cuda, half), _to_dev(g, cuda), _to_dev(b, cuda), _to_dev(emb, cuda, half)
                hw = shape[2] * shape[3]
                code = msd.DTYPE_F16 if half else msd.DTYPE_F32
                # the same whole-unit launch (same lanes, same vectors per lane) with one writer
                assert lib.msd_set_tuning(msd.TUNE_GN_SPLIT, 1) == 0
                assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, writers) == 0
                plan = msd.groupnorm_plan(shape[0], channels, hw, groups, code)
                assert plan[0] == 1 and plan[3] > 1, (shape, half, plan)
                assert msd.groupnorm_plan(shape[0], channels, hw, groups, code, in_place=True)[3] == 1
                assert lib.msd_set_tuning(msd.TUNE_GN_THREADS, plan[1]) == 0
                for silu in (True, False):
                    assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, 1) == 0
                    assert msd.groupnorm_plan(shape[0], channels, hw, groups, code) == plan[:3] + (1,)
                    one = msd.groupnorm(xd, gd, bd, groups, 1e-5, silu)
                    one_add = msd.chunk_add_groupnorm(xd, ed, gd, bd, groups, 1e-5, silu)
                    assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, writers) == 0
                    got = msd.groupnorm(xd, gd, bd, groups, 1e-5, silu)
                    got_add = msd.chunk_add_groupnorm(xd, ed, gd, bd, groups, 1e-5, silu)
                    assert torch.equal(got, one) and torch.equal(got_add, one_add), (shape, half, silu, plan)
                    z = xd.clone()
                    msd.groupnorm(z, gd, bd, groups, 1e-5, silu, out=z)   # in place: one writer
                    assert torch.equal(z, one), (shape, half, silu, "in place")
                assert lib.msd_set_tuning(msd.TUNE_GN_THREADS, 0) == 0
                assert lib.msd_set_tuning(msd.TUNE_GN_SPLIT, 0) == 0
                ref = orc.groupnorm(xin, g, b, groups, 1e-5, False)
                if half:
                    assert_close_f16(got.float().cpu().numpy(), ref, "gn writers f16 %s" % (shape,))
                else:
                    assert_close_f32(got.cpu().numpy(), ref, what="gn writers f32 %s" % (shape,))
    finally:
        assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, 0) == 0
        assert lib.msd_set_tuning(msd.TUNE_GN_THREADS, 0) == 0
        assert lib.msd_set_tuning(msd.TUNE_GN_SPLIT, 0) == 0
    # the knob is followed as far as every writer still owns a wavefront's vectors
    assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, writers) == 0
    try:
        assert msd.groupnorm_plan(2, 320, 4096, 32, msd.DTYPE_F16)[3] == writers
        assert msd.groupnorm_plan(2, 1280, 64, 32, msd.DTYPE_F16)[3] == min(writers, 4)   # 320 vectors: parts of 64 at least
    finally:
        assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, 0) == 0
    assert msd.status() == 0


@pytest.mark.parametrize("cus,xcds", [(256, 1), (64, 2), (128, 4), (512, 16), (228, 6)])
def test_groupnorm_planned_for_other_chips_runs_right_on_this_one(msd, orc, cuda, cus, xcds):
    """The launch follows the CU / XCD count the device reports; here other chips are injected
    through the knobs and the launches they get are run on the real device.  What changes is
    how many workgroups share a unit and how far apart their block ids are (one XCD count, any
    power of two; adjacent for one XCD or a count that is not a power of two): the result must
    not depend on it - equal to the oracle, and to the same launch with one writer bit for bit.
    Token-major store included (its block layout uses the same stride)."""
    torch = _torch()
    lib = msd.load_library()
    try:
        assert lib.msd_set_tuning(msd.TUNE_DEVICE_CUS, cus) == 0
        assert lib.msd_set_tuning(msd.TUNE_DEVICE_XCDS, xcds) == 0
        for batch, channels, hw, half in ((2, 640, 1024, True), (1, 1280, 256, True), (2, 320, 4096, False),
                                          (4, 1920, 256, True), (2, 1280, 64, False)):
            x = orc.normal((batch, channels, hw), seed=cus + xcds + channels, sigma=1.7, mean=0.2)
            g, b = _affine(orc, channels, cus + channels)
            code = msd.DTYPE_F16 if half else msd.DTYPE_F32
            plan = msd.groupnorm_plan(batch, channels, hw, 32, code)
            if plan[3] > 1:  # several writers: their stride is what the injected XCD count changes
                assert (batch * 32) % xcds == 0 and xcds & (xcds - 1) == 0 and batch * 32 * plan[3] <= cus
            xin = orc.round_to_half(x) if half else x
            xd, gd, bd = _to_dev(xin, cuda, half), _to_dev(g, cuda), _to_dev(b, cuda)
            got = msd.groupnorm(xd, gd, bd, 32, 1e-5, True)
            assert lib.msd_set_tuning(msd.TUNE_GN_THREADS, plan[1]) == 0
            assert lib.msd_set_tuning(msd.TUNE_GN_SPLIT, plan[0]) == 0
            assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, 1) == 0
            one = msd.groupnorm(xd, gd, bd, 32, 1e-5, True)
            for knob in (msd.TUNE_GN_THREADS, msd.TUNE_GN_SPLIT, msd.TUNE_GN_WRITERS):
                assert lib.msd_set_tuning(knob, 0) == 0
            if plan[3] > 1:
                assert torch.equal(got, one), (cus, xcds, batch, channels, hw, plan)
            ref = orc.groupnorm(xin, g, b, 32, 1e-5, True)
            if half:
                assert_close_f16(got.float().cpu().numpy(), ref, "gn other chip f16")
            else:
                assert_close_f32(got.cpu().numpy(), ref, what="gn other chip f32 %s" % ((cus, xcds, batch, channels, hw),))
            if channels <= 1280:  # token-major store of the same tensor (no SiLU, eps 1e-6)
                tok = msd.groupnorm_tokens(xd, gd, bd, 32, 1e-6).float().cpu().numpy()
                ref_t = np.ascontiguousarray(np.transpose(orc.groupnorm(xin, g, b, 32, 1e-6, False), (0, 2, 1)))
                if half:
                    assert_close_f16(tok, ref_t, "gn tokens other chip f16")
                else:
                    assert_close_f32(tok, ref_t, what="gn tokens other chip f32")
    finally:
        for knob in (msd.TUNE_DEVICE_CUS, msd.TUNE_DEVICE_XCDS, msd.TUNE_GN_THREADS, msd.TUNE_GN_SPLIT, msd.TUNE_GN_WRITERS):
            lib.msd_set_tuning(knob, 0)
    assert msd.status() == 0


def test_groupnorm_many_units_and_register_limits(msd, orc, cuda, gn_writers):
    # more units than scratch slots (never split), and float units that need a split to fit
    for shape, groups, half in [((300, 64, 4, 8), 32, True),     # 9600 units
                                ((1, 32, 64, 64), 2, False),     # 65536-element float units
                                ((2, 8, 128, 128), 1, False),    # 131072-element float units
                                ((1, 16, 256, 256), 1, True),    # 1 Mi-element half unit: 64 slices
                                ((1, 128, 256, 256), 32, True),  # decoder-sized map, 262144-element units
                                ((1, 128, 256, 256), 32, False),
                                ((1, 4, 512, 512), 2, False)]:   # 524288-element float units
        x = orc.normal(shape, seed=sum(shape), sigma=1.7, mean=-0.3)
        xin = orc.round_to_half(x) if half else x
        g, b = _affine(orc, shape[1], 41)
        ref = orc.groupnorm64(xin, g, b, groups, 1e-5, True)
        got = msd.groupnorm(_to_dev(xin, cuda, half), _to_dev(g, cuda), _to_dev(b, cuda), groups, 1e-5, True)
        got = got.float().cpu().numpy()
        if half:
            assert_close_f16(got, ref.astype(np.float32), "gn limits f16")
        else:
            assert_close_f32(got, ref, what="gn limits f32")
    assert msd.status() == 0


def test_shutdown_then_reuse(msd, orc, cuda):
    lib = msd.load_library()
    x = orc.normal((2, 320, 4096), seed=5, sigma=2.0)
    g, b = _affine(orc, 320, 5)
    _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, half=True)
    _torch().cuda.synchronize()
    assert lib.msd_shutdown() == 0
    _run_groupnorm(msd, orc, cuda, x, g, b, 32, 1e-5, True, half=True)  # scratch is created again
    assert msd.status() == 0
