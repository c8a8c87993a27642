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
    msd.gn_fallbacks(reset=True)  # bit-equality below holds while no workgroup gave up waiting for a sibling
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
        gave_up = msd.gn_fallbacks()
        assert torch.equal(got, want), "noalloc differs from msd_groupnorm at %s (msd_gn_fallbacks = %d)" % (
            (batch, channels, hw), gave_up)
        assert torch.equal(y, want), "noalloc in place differs from msd_groupnorm at %s (msd_gn_fallbacks = %d)" % (
            (batch, channels, hw), gave_up)
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


def test_noalloc_groupnorm_runs_under_stream_capture_and_allocates_nothing(msd, orc, cuda):
    """The callers the entry point is for: two calls of different shapes, both cut into slices
    that exchange through the fixed array, are recorded into one HIP graph (an allocation under
    capture would fail the capture), the device's free memory is the same after the calls as
    before, and every replay - with new input and the program's own eager work between replays -
    equals msd_groupnorm on the same input."""
    import torch
    lib = msd.load_library()
    code = msd.DTYPE_F16
    msd.init()  # the fixed array's address is looked up here, ahead of the capture
    msd.gn_fallbacks(reset=True)
    shapes = [(2, 320, 4096, 21), (1, 640, 1024, 22)]
    xs, gs, bs, gots, wants = [], [], [], [], []
    for batch, channels, hw, seed in shapes:
        xs.append(torch.from_numpy(orc.normal((batch, channels, hw), seed=seed, sigma=2.0)).to(cuda).half())
        gs.append(torch.from_numpy(orc.normal((channels,), seed=seed + 100, mean=1.0, sigma=0.1)).to(cuda))
        bs.append(torch.from_numpy(orc.normal((channels,), seed=seed + 200, sigma=0.1)).to(cuda))
        gots.append(torch.zeros_like(xs[-1]))
        wants.append(torch.empty_like(xs[-1]))
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    try:
        assert lib.msd_set_tuning(msd.TUNE_GN_SPLIT, 4) == 0
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        sp = torch.cuda.current_stream().cuda_stream
        for (batch, channels, hw, _), x, g, b, got in zip(shapes, xs, gs, bs, gots):
            assert _call(lib.msd_groupnorm_noalloc, x, got, g, b, batch, channels, hw, True, code, sp) == 0
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "msd_groupnorm_noalloc changed the device's free memory"
        for got in gots:
            got.zero_()
        with torch.cuda.graph(graph, stream=side):
            sp = torch.cuda.current_stream().cuda_stream
            for (batch, channels, hw, _), x, g, b, got in zip(shapes, xs, gs, bs, gots):
                assert _call(lib.msd_groupnorm_noalloc, x, got, g, b, batch, channels, hw, True, code, sp) == 0
        torch.cuda.synchronize()
        for replay in range(3):
            for x in xs:  # new input for every replay, written eagerly
                x.mul_(0.5).add_(0.25 * replay)
            graph.replay()
            torch.cuda.synchronize()
            sp = torch.cuda.current_stream().cuda_stream
            for (batch, channels, hw, _), x, g, b, want in zip(shapes, xs, gs, bs, wants):
                assert _call(lib.msd_groupnorm, x, want, g, b, batch, channels, hw, True, code, sp) == 0
            torch.cuda.synchronize()
            gave_up = msd.gn_fallbacks()
            for got, want, shape in zip(gots, wants, shapes):
                assert torch.equal(got, want), "replay %d differs from msd_groupnorm at %s (msd_gn_fallbacks = %d)" % (
                    replay, shape[:3], gave_up)
    finally:
        lib.msd_set_tuning(msd.TUNE_GN_SPLIT, 0)
