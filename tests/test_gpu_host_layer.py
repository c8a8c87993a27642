"""The C++ layer objects on the GPU, used the way the reference uses its own: weights come
from .npy files under the media path, init() loads them, forward(input, output) runs, and
the result is checked against a golden .npy with util::testBuffer (here the golden file is
written from the CPU oracle's output)."""
import ctypes

import numpy as np
import pytest

from tolerances import assert_close_f16, assert_close_f32

pytestmark = pytest.mark.gpu


@pytest.fixture()
def nn(msd, tmp_path, cuda):
    lib = msd.load_nn_library()
    lib.msdnn_set_media_path(str(tmp_path).encode())
    return lib


def _dev(a, cuda, half=False):
    import torch
    t = torch.from_numpy(np.ascontiguousarray(a)).to(cuda)
    return t.half() if half else t


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _test_buffer(nn, t, golden_name):
    md, nw = ctypes.c_float(0), ctypes.c_size_t(0)
    code = 1 if t.element_size() == 2 else 0
    rc = nn.msdnn_test_buffer(None, _ptr(t), t.numel() * t.element_size(), code, golden_name.encode(),
                              ctypes.byref(md), ctypes.byref(nw))
    return rc, md.value, nw.value


@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
def test_groupnorm_object_like_resblock(msd, nn, orc, cuda, tmp_path, half):
    import torch
    channels, side, batch = 320, 32, 2
    w = orc.normal((channels,), seed=11, mean=1.0, sigma=0.1)
    b = orc.normal((channels,), seed=12, sigma=0.1)
    np.save(tmp_path / "in_norm_weight.npy", w)
    np.save(tmp_path / "in_norm_bias.npy", b)
    x = orc.normal((batch, channels, side, side), seed=13, sigma=2.0)
    xin = orc.round_to_half(x) if half else x
    ref = orc.groupnorm(xin, w, b, 32, 1e-5, silu=True)
    np.save(tmp_path / "golden.npy", orc.round_to_half(ref) if half else ref)
    g = nn.msdnn_groupnorm_create(None, 32, channels, 1e-5, b"in_norm_weight.npy", b"in_norm_bias.npy", batch, 1)
    assert g and nn.msdnn_groupnorm_init(g) == 0, msd.nn_last_error()
    assert nn.msdnn_groupnorm_init(g) == 0  # idempotent (M/nn/GroupNorm.cpp:52-54)
    xd = _dev(xin, cuda, half)
    yd = torch.empty_like(xd)
    nbytes = xd.numel() * xd.element_size()
    assert nn.msdnn_groupnorm_forward(g, _ptr(xd), _ptr(yd), nbytes, int(half)) == 0, msd.nn_last_error()
    rc, max_diff, _ = _test_buffer(nn, yd, "golden.npy")
    assert rc == 0
    got = yd.float().cpu().numpy()
    if half:
        assert_close_f16(got, orc.round_to_half(ref))
    else:
        assert_close_f32(got, ref)
        assert max_diff < 1e-5  # the reference logged 9.5e-7 .. 7.3e-6 for these checks
    # in place, as the out-norm of a ResBlock (M/nn/ResBlock.cpp:222)
    assert nn.msdnn_groupnorm_forward(g, _ptr(xd), _ptr(xd), nbytes, int(half)) == 0
    assert torch.equal(xd, yd)
    # precondition failures surface as errors, not launches
    assert nn.msdnn_groupnorm_forward(g, _ptr(xd), _ptr(yd), nbytes - 2 * xd.element_size(), int(half)) < 0
    nn.msdnn_groupnorm_destroy(g)
    assert msd.status() == 0


def test_layernorm_geglu_objects_like_transformer_block(msd, nn, orc, cuda, tmp_path):
    import torch
    dim, rows = 320, 2 * 1024
    w = orc.normal((dim,), seed=21, mean=1.0, sigma=0.1)
    b = orc.normal((dim,), seed=22, sigma=0.1)
    np.save(tmp_path / "norm3_weight.npy", w)
    np.save(tmp_path / "norm3_bias.npy", b)
    x = orc.normal((rows, dim), seed=23)
    ref = orc.layernorm(x, w, b, 1e-5)
    np.save(tmp_path / "test_basic_norm_3.npy", ref)
    ln = nn.msdnn_layernorm_create(None, dim, b"norm3_weight.npy", b"norm3_bias.npy", 1e-5)
    assert nn.msdnn_layernorm_init(ln) == 0, msd.nn_last_error()
    xd = _dev(x, cuda)
    yd = torch.empty_like(xd)
    assert nn.msdnn_layernorm_forward(ln, _ptr(xd), _ptr(yd), x.nbytes, 0) == 0
    rc, max_diff, _ = _test_buffer(nn, yd, "test_basic_norm_3.npy")
    assert rc == 0 and max_diff < 1e-5  # the reference logged 4.77e-6 here
    assert_close_f32(yd.cpu().numpy(), ref)
    nn.msdnn_layernorm_destroy(ln)

    ge = nn.msdnn_geglu_create(None, dim, 4 * dim)
    proj = orc.round_to_half(orc.normal((rows, 8 * dim), seed=24))
    refg = orc.round_to_half(orc.geglu(proj))
    pd = _dev(proj, cuda, True)
    od = torch.empty((rows, 4 * dim), dtype=torch.float16, device=cuda)
    assert nn.msdnn_geglu_forward(ge, _ptr(pd), pd.numel() * 2, _ptr(od), od.numel() * 2, 1) == 0
    assert_close_f16(od.float().cpu().numpy(), refg)
    assert nn.msdnn_geglu_forward(ge, _ptr(pd), pd.numel() * 2, _ptr(od), od.numel() * 2 - 2, 1) < 0
    nn.msdnn_geglu_destroy(ge)


def test_activations_and_timestep_embedding_through_objects(msd, nn, orc, cuda):
    import torch
    x = orc.normal((2, 1280), seed=31, sigma=2.0)
    for op, ref_fn in ((0, orc.silu), (1, orc.gelu), (2, orc.quick_gelu)):
        xd = _dev(x, cuda)
        assert nn.msdnn_activation(None, op, _ptr(xd), _ptr(xd), x.nbytes, 0) == 0  # in place
        assert_close_f32(xd.cpu().numpy(), ref_fn(x))
    # the timestep the shipped app uses (native-lib.cpp:240) and a CFG pair
    for ts in ([981], [961, 961], [0, 999]):
        arr = (ctypes.c_long * len(ts))(*ts)
        out = (ctypes.c_float * (len(ts) * 320))()
        assert nn.msdnn_timestep_embedding(None, arr, len(ts), out) == 0, msd.nn_last_error()
        got = np.array(out[:], dtype=np.float32).reshape(len(ts), 320)
        ref = np.stack([orc.timestep_embedding(t) for t in ts])
        assert_close_f32(got, ref)
    torch.cuda.synchronize()


def test_objects_with_fused_adds(msd, nn, orc, cuda, tmp_path):
    """ResBlock out-norm with the embedding add, and LayerNorm 2 with the residual add, through
    the layer objects (M/nn/ResBlock.cpp:188-232, M/nn/BasicTransformerBlock.cpp:126-136)."""
    import torch
    channels, hw, batch = 640, 1024, 2
    w = orc.normal((channels,), seed=41, mean=1.0, sigma=0.1)
    b = orc.normal((channels,), seed=42, sigma=0.1)
    np.save(tmp_path / "out_w.npy", w)
    np.save(tmp_path / "out_b.npy", b)
    x = orc.round_to_half(orc.normal((batch, channels, hw), seed=43, sigma=1.5))
    emb = orc.round_to_half(orc.normal((batch, channels), seed=44))
    g = nn.msdnn_groupnorm_create(None, 32, channels, 1e-5, b"out_w.npy", b"out_b.npy", batch, 1)
    assert nn.msdnn_groupnorm_init(g) == 0, msd.nn_last_error()
    xd, ed = _dev(x, cuda, True), _dev(emb, cuda, True)
    nbytes = xd.numel() * 2
    assert nn.msdnn_groupnorm_forward_chunk(g, _ptr(xd), _ptr(ed), ed.numel() * 2, _ptr(xd), nbytes, 1) == 0
    ref = orc.groupnorm(orc.round_to_half(orc.chunkwise_add(x, emb, hw)), w, b, 32, 1e-5, silu=True)
    assert_close_f16(xd.float().cpu().numpy(), orc.round_to_half(ref))
    assert nn.msdnn_groupnorm_forward_chunk(g, _ptr(xd), _ptr(ed), ed.numel() * 2 - 2, _ptr(xd), nbytes, 1) < 0
    assert "chunk size" in msd.nn_last_error()
    nn.msdnn_groupnorm_destroy(g)

    # SpatialTransformer's norm (eps 1e-6, no SiLU) written token-major (M/nn/SpatialTransformer.cpp:127-139)
    g = nn.msdnn_groupnorm_create(None, 32, channels, 1e-6, b"out_w.npy", b"out_b.npy", batch, 0)
    assert nn.msdnn_groupnorm_init(g) == 0, msd.nn_last_error()
    xd = _dev(x, cuda, True)
    td = torch.empty((batch, hw, channels), dtype=torch.float16, device=cuda)
    assert nn.msdnn_groupnorm_forward_tokens(g, _ptr(xd), _ptr(td), nbytes, 1) == 0, msd.nn_last_error()
    ref = orc.groupnorm(x, w, b, 32, 1e-6, silu=False)
    assert_close_f16(td.float().cpu().numpy(), orc.round_to_half(ref).transpose(0, 2, 1))
    assert nn.msdnn_groupnorm_forward_tokens(g, _ptr(xd), _ptr(xd), nbytes, 1) < 0  # needs separate output
    nn.msdnn_groupnorm_destroy(g)

    dim, rows = 640, 2048
    lw = orc.normal((dim,), seed=45, mean=1.0, sigma=0.1)
    lb = orc.normal((dim,), seed=46, sigma=0.1)
    np.save(tmp_path / "n2_w.npy", lw)
    np.save(tmp_path / "n2_b.npy", lb)
    a = orc.normal((rows, dim), seed=47)
    r = orc.normal((rows, dim), seed=48, sigma=2.0)
    ln = nn.msdnn_layernorm_create(None, dim, b"n2_w.npy", b"n2_b.npy", 1e-5)
    assert nn.msdnn_layernorm_init(ln) == 0, msd.nn_last_error()
    ad, rd = _dev(a, cuda), _dev(r, cuda)
    yd = torch.empty_like(ad)
    assert nn.msdnn_layernorm_forward_add(ln, _ptr(ad), _ptr(rd), _ptr(ad), _ptr(yd), a.nbytes, 0) == 0
    s = orc.elemwise_add(a, r)
    assert np.array_equal(ad.cpu().numpy(), s)  # the sum replaced the first operand
    assert_close_f32(yd.cpu().numpy(), orc.layernorm(s, lw, lb, 1e-5))
    nn.msdnn_layernorm_destroy(ln)


def test_step_runner_eager_and_graph(msd, nn, cuda):
    import torch
    stream = torch.cuda.Stream()  # graph capture needs a stream of its own, not the default one
    st = nn.msdnn_step_create(ctypes.c_void_p(stream.cuda_stream), 2, 1)
    assert st, msd.nn_last_error()
    assert nn.msdnn_step_bytes(st) == 1099694080  # 45 GroupNorm + 48 LayerNorm + 16 GEGLU, fp16, batch 2
    assert nn.msdnn_step_launches(st) == 133
    ts = (ctypes.c_long * 2)(961, 961)
    assert nn.msdnn_step_run(st, 2, 0, ts, 2) == 0, msd.nn_last_error()
    assert nn.msdnn_step_run(st, 3, 1, ts, 2) == 0, msd.nn_last_error()
    torch.cuda.synchronize()
    assert msd.load_library().msd_status(ctypes.c_void_p(stream.cuda_stream)) == 0
    nn.msdnn_step_destroy(st)
    # the default stream cannot be captured: reported, not crashed
    st0 = nn.msdnn_step_create(None, 1, 0)
    assert nn.msdnn_step_run(st0, 1, 1, (ctypes.c_long * 1)(5), 1) < 0
    assert "non-default stream" in msd.nn_last_error()
    assert nn.msdnn_step_run(st0, 1, 0, (ctypes.c_long * 1)(5), 1) == 0
    torch.cuda.synchronize()
    nn.msdnn_step_destroy(st0)
