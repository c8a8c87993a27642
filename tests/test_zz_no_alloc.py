"""msd_groupnorm_noalloc (the entry point that allocates nothing: its workgroups exchange
partial statistics through a fixed array inside the library's code object) against
msd_groupnorm (per-stream allocated scratch), through the C ABI: same bits, on two calls in a
row, the second with a smaller input, so that whatever the first call left in the shared array
is still there when the second one runs."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _call(fn, x, y, g, b, batch, channels, hw, silu, code, stream):
    vp = ctypes.c_void_p
    return fn(vp(x.data_ptr()), vp(y.data_ptr()), vp(g.data_ptr()), vp(b.data_ptr()), batch, channels, hw, 32,
              1e-5, int(silu), code, vp(stream))


@pytest.mark.parametrize("half", [True, False], ids=["f16", "f32"])
def test_noalloc_groupnorm_matches_allocating_entry_point_twice(msd, orc, cuda, half):
    import torch
    lib = msd.load_library()
    code = msd.DTYPE_F16 if half else msd.DTYPE_F32
    stream = torch.cuda.current_stream().cuda_stream
    # both shapes are cut into several workgroups per (sample, group), so both calls use the
    # exchange area; the second is smaller (fewer units, shorter slices)
    for batch, channels, hw, seed in [(2, 320, 4096, 11), (1, 640, 1024, 12)]:
        x = orc.normal((batch, channels, hw), seed=seed, sigma=2.0, mean=0.3)
        g = orc.normal((channels,), seed=seed + 100, mean=1.0, sigma=0.1)
        b = orc.normal((channels,), seed=seed + 200, sigma=0.1)
        xd = torch.from_numpy(x).to(cuda)
        xd = xd.half() if half else xd
        gd, bd = torch.from_numpy(g).to(cuda), torch.from_numpy(b).to(cuda)
        want = torch.empty_like(xd)
        got = torch.zeros_like(xd)
        try:
            assert lib.msd_set_tuning(msd.TUNE_GN_SPLIT, 4) == 0  # the exchange is used at both sizes
            assert _call(lib.msd_groupnorm, xd, want, gd, bd, batch, channels, hw, True, code, stream) == 0
            assert _call(lib.msd_groupnorm_noalloc, xd, got, gd, bd, batch, channels, hw, True, code, stream) == 0
            # in place, as the reference's out-norm runs (M/nn/ResBlock.cpp:222): one more call on the same array
            y = xd.clone()
            assert _call(lib.msd_groupnorm_noalloc, y, y, gd, bd, batch, channels, hw, True, code, stream) == 0
        finally:
            lib.msd_set_tuning(msd.TUNE_GN_SPLIT, 0)
        torch.cuda.synchronize()
        assert torch.equal(got, want), "noalloc differs from msd_groupnorm at %s" % ((batch, channels, hw),)
        assert torch.equal(y, want), "noalloc in place differs from msd_groupnorm at %s" % ((batch, channels, hw),)
        # and both are right: the oracle on the same input
        from tolerances import assert_close_f16, assert_close_f32
        xin = xd.float().cpu().numpy()
        ref = orc.groupnorm(xin, g, b, 32, 1e-5, silu=True)
        if half:
            assert_close_f16(got.float().cpu().numpy(), ref, "noalloc groupnorm f16")
        else:
            assert_close_f32(got.cpu().numpy(), ref, what="noalloc groupnorm f32")
    # with the automatic launch plan too (whatever it picks, both entry points pick the same)
    assert _call(lib.msd_groupnorm, xd, want, gd, bd, batch, channels, hw, True, code, stream) == 0
    assert _call(lib.msd_groupnorm_noalloc, xd, got, gd, bd, batch, channels, hw, True, code, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    # beyond the fixed array: refused with the dedicated code, nothing launched
    assert _call(lib.msd_groupnorm_noalloc, xd, got, gd, bd, 40, channels, hw, True, code, stream) == msd.ERR_SCRATCH_LIMIT
