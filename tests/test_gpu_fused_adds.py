"""The two additions the reference runs in front of its norms (chunkwise_add before the
ResBlock out-norm, elemwise_add before LayerNorm 2 / 3) and their fusion into the norm
kernels.  Fused launches must equal the two-launch sequence bit for bit, and both must match
the CPU oracle's restatement of the reference kernels."""
import ctypes

import numpy as np
import pytest

from tolerances import assert_close_f16, assert_close_f32, assert_one_ulp16_apart

pytestmark = pytest.mark.gpu


def _dev(a, cuda, half=False):
    import torch
    t = torch.from_numpy(np.ascontiguousarray(a)).to(cuda)
    return t.half() if half else t


def _affine(orc, n, seed):
    return (orc.normal((n,), seed=seed, mean=1.0, sigma=0.1), orc.normal((n,), seed=seed + 1, sigma=0.1))


@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
@pytest.mark.parametrize("n,chunk", [(2 * 320 * 1024, 1024), (3 * 7 * 9, 9), (1031, 0), (2 * 4096 * 320, 0), (40, 8)])
def test_add_kernels(msd, orc, cuda, n, chunk, half):
    a = orc.normal((n,), seed=n, sigma=2.0)
    if chunk:
        b = orc.normal((n // chunk,), seed=n + 1)
    else:
        b = orc.normal((n,), seed=n + 1)
    ain, bin_ = (orc.round_to_half(a), orc.round_to_half(b)) if half else (a, b)
    ref = orc.chunkwise_add(ain, bin_, chunk) if chunk else orc.elemwise_add(ain, bin_)
    ad, bd = _dev(ain, cuda, half), _dev(bin_, cuda, half)
    got = msd.chunkwise_add(ad, bd, chunk, out=ad) if chunk else msd.elemwise_add(ad, bd, out=ad)  # in place
    got = got.float().cpu().numpy()
    if half:
        assert np.array_equal(got, orc.round_to_half(ref))  # one rounding of an exact sum
    else:
        assert np.array_equal(got, ref)


@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
@pytest.mark.parametrize("shape,groups", [((2, 320, 64, 64), 32), ((2, 640, 32, 32), 32), ((2, 1280, 8, 8), 32),
                                          ((1, 96, 24, 24), 32), ((3, 64, 5, 7), 8), ((1, 8, 128, 128), 1)])
def test_chunk_add_groupnorm_equals_two_launches(msd, orc, cuda, shape, groups, half):
    import torch
    batch, channels = shape[0], shape[1]
    hw = int(np.prod(shape[2:]))
    x = orc.normal(shape, seed=sum(shape), sigma=1.5)
    emb = orc.normal((batch, channels), seed=sum(shape) + 1, sigma=0.7)
    g, b = _affine(orc, channels, 7)
    xin, ein = (orc.round_to_half(x), orc.round_to_half(emb)) if half else (x, emb)
    xd, ed, gd, bd = _dev(xin, cuda, half), _dev(ein, cuda, half), _dev(g, cuda), _dev(b, cuda)
    fused = msd.chunk_add_groupnorm(xd, ed, gd, bd, groups, 1e-5, True)
    tmp = msd.chunkwise_add(xd, ed, hw)
    two = msd.groupnorm(tmp, gd, bd, groups, 1e-5, True)
    assert torch.equal(fused, two)
    # in place, as the reference runs its out-norm (M/nn/ResBlock.cpp:222): the launch never lets
    # several workgroups share a unit then, so it is compared with the same launch out of place
    lib = msd.load_library()
    assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, 1) == 0
    try:
        apart = msd.chunk_add_groupnorm(xd.clone(), ed, gd, bd, groups, 1e-5, True)
    finally:
        assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, 0) == 0
    xc = xd.clone()
    assert torch.equal(msd.chunk_add_groupnorm(xc, ed, gd, bd, groups, 1e-5, True, out=xc), apart)
    # oracle: chunkwise_add, (storage rounding), group norm, silu
    s = orc.chunkwise_add(xin, ein, hw)
    if half:
        s = orc.round_to_half(s)
    ref = orc.groupnorm64(s, g, b, groups, 1e-5, True)
    got = fused.float().cpu().numpy()
    if half:
        assert_close_f16(got, ref.astype(np.float32), "chunk add gn f16")
    else:
        assert_close_f32(got, ref, what="chunk add gn f32")
    assert msd.status() == 0


@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
@pytest.mark.parametrize("rows,dim", [(8192, 320), (2048, 640), (512, 1280), (77, 1024), (5, 100), (9, 64)])
def test_add_layernorm_equals_two_launches(msd, orc, cuda, rows, dim, half):
    import torch
    a = orc.normal((rows, dim), seed=rows + dim, sigma=1.2)
    r = orc.normal((rows, dim), seed=rows + dim + 1, sigma=0.8, mean=0.5)
    g, b = _affine(orc, dim, 9)
    ain, rin = (orc.round_to_half(a), orc.round_to_half(r)) if half else (a, r)
    ad, rd, gd, bd = _dev(ain, cuda, half), _dev(rin, cuda, half), _dev(g, cuda), _dev(b, cuda)
    s_fused, y_fused = msd.add_layernorm(ad, rd, gd, bd)
    s_two = msd.elemwise_add(ad, rd)
    y_two = msd.layernorm(s_two, gd, bd)
    assert torch.equal(s_fused, s_two) and torch.equal(y_fused, y_two)
    # sum written over the first operand, as M/nn/BasicTransformerBlock.cpp:126-134 does
    ac = ad.clone()
    s_in, y_in = msd.add_layernorm(ac, rd, gd, bd, sum_out=ac)
    assert s_in.data_ptr() == ac.data_ptr() and torch.equal(s_in, s_two) and torch.equal(y_in, y_two)
    s_ref = orc.elemwise_add(ain, rin)
    if half:
        s_ref = orc.round_to_half(s_ref)
    ref = orc.layernorm64(s_ref, g, b, 1e-5)
    got = y_fused.float().cpu().numpy()
    if half:
        assert np.array_equal(s_fused.float().cpu().numpy(), s_ref)
        assert_close_f16(got, ref.astype(np.float32), "add ln f16")
    else:
        assert np.array_equal(s_fused.cpu().numpy(), s_ref)
        assert_close_f32(got, ref, what="add ln f32")


@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
@pytest.mark.parametrize("shape,groups,split", [((2, 320, 64, 64), 32, 0), ((2, 640, 32, 32), 32, 0),
                                                ((2, 1280, 16, 16), 32, 0), ((2, 1280, 8, 8), 32, 0),
                                                ((1, 320, 64, 64), 32, 8), ((2, 640, 32, 32), 32, 2),
                                                ((1, 96, 24, 24), 32, 0), ((3, 64, 5, 7), 8, 0),
                                                ((1, 33, 4, 4), 33, 0), ((1, 8, 128, 128), 1, 0),
                                                ((8, 320, 32, 32), 32, 0), ((4, 640, 32, 32), 32, 0)])
@pytest.mark.parametrize("writers", [0, 1, 4, 16], ids=["writers-auto", "one-writer", "4-writers", "16-writers"])
def test_groupnorm_tokens_equals_norm_then_permute(msd, orc, cuda, shape, groups, split, half, writers):
    """SpatialTransformer's GroupNorm(eps 1e-6, no SiLU) + permute (0, 2, 1) in one launch
    (M/nn/SpatialTransformer.cpp:127-139): slices of positions with an exchange, or (writers != 1,
    where the shape allows it) several workgroups that each reduce the whole unit and store the
    tokens of one range of positions."""
    import torch
    lib = msd.load_library()
    batch, channels = shape[0], shape[1]
    hw = int(np.prod(shape[2:]))
    x = orc.normal(shape, seed=sum(shape) + 3, sigma=1.5, mean=0.4)
    g, b = _affine(orc, channels, 11)
    xin = orc.round_to_half(x) if half else x
    xd, gd, bd = _dev(xin, cuda, half), _dev(g, cuda), _dev(b, cuda)
    try:
        lib.msd_set_tuning(msd.TUNE_GN_SPLIT, split)
        assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, writers) == 0
        fused = msd.groupnorm_tokens(xd, gd, bd, groups, 1e-6)
    finally:
        lib.msd_set_tuning(msd.TUNE_GN_SPLIT, 0)
        lib.msd_set_tuning(msd.TUNE_GN_WRITERS, 0)
    two = msd.groupnorm(xd, gd, bd, groups, 1e-6, False).view(batch, channels, hw).permute(0, 2, 1).contiguous()
    assert fused.shape == (batch, hw, channels)
    # the slices cut positions instead of channel ranges, so the statistics are summed in another
    # order: equal to the two-launch result up to that (a few float ulps), not bit for bit
    d = (fused.float() - two.float()).abs()
    if half:
        assert (d == 0).float().mean().item() > 0.999
        assert_one_ulp16_apart(fused.float().cpu().numpy(), two.float().cpu().numpy(), "gn tokens vs two launches")
    else:
        assert (d / two.abs().clamp(min=1.0)).max().item() < 2e-6
    ref = np.concatenate([orc.permute_0_2_1(orc.groupnorm64(xin, g, b, groups, 1e-6, False)
                                            .astype(np.float32).reshape(batch, channels, hw)[i:i + 1])
                          for i in range(batch)])
    got = fused.float().cpu().numpy()
    if half:
        assert_close_f16(got, ref, "gn tokens f16")
    else:
        assert_close_f32(got, ref, what="gn tokens f32")
    assert msd.status() == 0


@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
@pytest.mark.parametrize("shape", [(2, 320, 4096), (2, 4096, 320), (1, 1280, 64), (3, 100, 36), (2, 7, 5),
                                   (1, 64, 64), (5, 68, 132), (1, 1, 8),
                                   # 16-byte pieces on both sides with ragged tiles, one tile, thin planes
                                   (3, 72, 200), (2, 8, 8), (1, 136, 64), (2, 16, 1000), (4, 264, 24)])
def test_permute_0_2_1(msd, orc, cuda, shape, half):
    import torch
    x = orc.normal(shape, seed=sum(shape))
    xin = orc.round_to_half(x) if half else x
    got = msd.permute_0_2_1(_dev(xin, cuda, half))
    assert np.array_equal(got.float().cpu().numpy(), orc.permute_0_2_1(xin))
    assert torch.equal(msd.permute_0_2_1(got), _dev(xin, cuda, half))  # its own inverse


def test_fused_argument_checks(msd, cuda):
    lib = msd.load_library()
    assert lib.msd_chunk_add_groupnorm(None, None, None, None, None, 1, 32, 16, 32, 1e-5, 0, 0, None) == 1
    assert lib.msd_add_layernorm(None, None, None, None, None, None, 4, 64, 1e-5, 0, None) == 1
    assert lib.msd_chunkwise_add(None, None, None, 16, 0, 0, None) == 1
    assert lib.msd_elemwise_add(None, None, None, 0, 0, None) == 0
    import torch
    x = torch.zeros(32 * 64, device=cuda)
    p = ctypes.c_void_p(x.data_ptr())
    assert lib.msd_groupnorm_tokens(p, p, p, p, 1, 32, 64, 32, 1e-6, 0, None) == 1  # y must not be x
