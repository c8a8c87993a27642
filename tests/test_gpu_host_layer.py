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
        assert_close_f16(got, ref)
    else:
        assert_close_f32(got, ref)
        assert max_diff < 1e-5  # the reference logged 9.5e-7 .. 7.3e-6 for these checks
    # in place, as the out-norm of a ResBlock (M/nn/ResBlock.cpp:222).  Such a call never lets several
    # workgroups share a unit, so its bits are those of the same launch out of place; against the
    # shared launch above only the summation order differs
    lib = msd.load_library()
    one = torch.empty_like(xd)
    assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, 1) == 0
    try:
        assert nn.msdnn_groupnorm_forward(g, _ptr(xd), _ptr(one), nbytes, int(half)) == 0
    finally:
        assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, 0) == 0
    assert nn.msdnn_groupnorm_forward(g, _ptr(xd), _ptr(xd), nbytes, int(half)) == 0
    assert torch.equal(xd, one)
    if half:
        assert (xd == yd).float().mean().item() > 0.999
    else:
        assert ((xd - yd).abs() / yd.abs().clamp(min=1.0)).max().item() < 2e-6
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
    refg = orc.geglu(proj)
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
    assert_close_f16(xd.float().cpu().numpy(), ref)
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
    assert_close_f16(td.float().cpu().numpy(), ref.transpose(0, 2, 1))
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
    st = nn.msdnn_step_create(ctypes.c_void_p(stream.cuda_stream), 2, 1, 0)
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
    st0 = nn.msdnn_step_create(None, 1, 0, 0)
    assert nn.msdnn_step_run(st0, 1, 1, (ctypes.c_long * 1)(5), 1) < 0
    assert "non-default stream" in msd.nn_last_error()
    assert nn.msdnn_step_run(st0, 1, 0, (ctypes.c_long * 1)(5), 1) == 0
    torch.cuda.synchronize()
    nn.msdnn_step_destroy(st0)


# ----------------------------------------------------------------- neighbours of the path
@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
def test_linear_objects_grouped_forward_equals_one_call_per_layer(msd, nn, orc, cuda, half):
    """Linear::forwardSiluGrouped: the embed_linear of several ResBlocks on the same emb in one
    launch (M/nn/ResBlock.cpp:173-183), bit for bit what each layer's own forwardSilu gives."""
    import ctypes
    import torch
    couts = [320, 640, 1280, 1280, 640]
    fp = ctypes.POINTER(ctypes.c_float)
    dt = torch.float16 if half else torch.float32
    es = 2 if half else 4
    layers = []
    for i, n in enumerate(couts):
        l = nn.msdnn_linear_create(None, 1280, n, None, None, int(half))
        w = orc.normal((n, 1280), seed=700 + i, sigma=1280 ** -0.5)
        b = orc.normal((n,), seed=720 + i, sigma=0.1)
        assert l and nn.msdnn_linear_init_from(l, w.ctypes.data_as(fp), w.size, b.ctypes.data_as(fp), b.size) == 0
        layers.append(l)
    emb = torch.randn((2, 1280), device=cuda, generator=torch.Generator(device=cuda).manual_seed(5)).to(dt)
    single = [torch.empty((2, n), dtype=dt, device=cuda) for n in couts]
    grouped = [torch.empty((2, n), dtype=dt, device=cuda) for n in couts]
    try:
        for l, o in zip(layers, single):
            assert nn.msdnn_linear_forward(l, _ptr(emb), emb.numel() * es, _ptr(o), o.numel() * es, int(half), 1, 0) == 0
        hs = (ctypes.c_void_p * len(layers))(*layers)
        outs = (ctypes.c_void_p * len(layers))(*[o.data_ptr() for o in grouped])
        nbytes = (ctypes.c_size_t * len(layers))(*[o.numel() * es for o in grouped])
        assert nn.msdnn_linear_forward_grouped(hs, len(layers), _ptr(emb), emb.numel() * es, outs, nbytes, int(half),
                                               1, 0) == 0, msd.nn_last_error()
        torch.cuda.synchronize()
        for a, b in zip(single, grouped):
            assert torch.equal(a, b)
        # refusals: one output per layer with the layer's size; the input is not an output
        nbytes[1] = 16
        assert nn.msdnn_linear_forward_grouped(hs, len(layers), _ptr(emb), emb.numel() * es, outs, nbytes, int(half),
                                               1, 0) < 0
        assert "output size" in msd.nn_last_error()
    finally:
        for l in layers:
            nn.msdnn_linear_destroy(l)


@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
def test_linear_objects_run_the_time_embedding_mlp(msd, nn, orc, cuda, tmp_path, half):
    """time_embed_0 + SiLU, time_embed_2, then a ResBlock's SiLU + embed_linear, weights from .npy."""
    import torch
    shapes = {"time_embed_0": (1280, 320), "time_embed_2": (1280, 1280), "embed_linear": (640, 1280)}
    weights = {}
    for i, (name, (n, k)) in enumerate(shapes.items()):
        w = orc.normal((n, k), seed=300 + i, sigma=k ** -0.5)
        b = orc.normal((n,), seed=310 + i, sigma=0.1)
        np.save(tmp_path / (name + "_weight.npy"), w)
        np.save(tmp_path / (name + "_bias.npy"), b)
        weights[name] = (orc.round_to_half(w) if half else w, b)
    temb = np.stack([orc.timestep_embedding(t) for t in (981, 21)])
    temb = orc.round_to_half(temb) if half else temb
    rnd = orc.round_to_half if half else (lambda v: v)
    h = rnd(orc.silu(orc.linear(temb, *weights["time_embed_0"])))
    emb = rnd(orc.linear(h, *weights["time_embed_2"]))
    ref = rnd(orc.linear(orc.silu(emb), *weights["embed_linear"]))

    layers = {}
    for name, (n, k) in shapes.items():
        l = nn.msdnn_linear_create(None, k, n, (name + "_weight.npy").encode(), (name + "_bias.npy").encode(),
                                   int(half))
        assert l and nn.msdnn_linear_init(l) == 0, msd.nn_last_error()
        layers[name] = l
    dt = torch.float16 if half else torch.float32
    es = 2 if half else 4
    x = _dev(temb, cuda, half)
    hd = torch.empty((2, 1280), dtype=dt, device=cuda)
    ed = torch.empty((2, 1280), dtype=dt, device=cuda)
    od = torch.empty((2, 640), dtype=dt, device=cuda)
    fw = nn.msdnn_linear_forward
    assert fw(layers["time_embed_0"], _ptr(x), 2 * 320 * es, _ptr(hd), 2 * 1280 * es, int(half), 0, 1) == 0
    assert fw(layers["time_embed_2"], _ptr(hd), 2 * 1280 * es, _ptr(ed), 2 * 1280 * es, int(half), 0, 0) == 0
    assert fw(layers["embed_linear"], _ptr(ed), 2 * 1280 * es, _ptr(od), 2 * 640 * es, int(half), 1, 0) == 0
    if half:
        # layer by layer: each stored fp16 result against the oracle applied to the stored fp16
        # input the layer actually saw (a rounding flip upstream is then not this layer's error)
        h_gpu, e_gpu = hd.float().cpu().numpy(), ed.float().cpu().numpy()
        assert_close_f16(h_gpu, orc.silu(orc.linear(temb, *weights["time_embed_0"])), "time_embed_0 f16")
        assert_close_f16(e_gpu, orc.linear(h_gpu, *weights["time_embed_2"]), "time_embed_2 f16")
        assert_close_f16(od.float().cpu().numpy(), orc.linear(orc.silu(e_gpu), *weights["embed_linear"]),
                         "embed_linear f16")
        # and the chain as a whole stays within a few fp16 ulps of the all-oracle chain
        np.testing.assert_allclose(od.float().cpu().numpy(), ref, atol=4e-3, rtol=2e-3)
    else:
        assert_close_f32(ed.cpu().numpy(), emb, what="time_embed")
        assert_close_f32(od.cpu().numpy(), ref, what="embed_linear")
    # the reference's refusals (M/nn/Linear.cpp:78-92)
    assert fw(layers["time_embed_2"], _ptr(hd), 2 * 1280 * es, _ptr(hd), 2 * 1280 * es, int(half), 0, 0) < 0
    assert msd.nn_last_error() == "Linear not support input == output"
    assert fw(layers["time_embed_2"], _ptr(hd), (2 * 1280 - 1) * es, _ptr(ed), 2 * 1280 * es, int(half), 0, 0) < 0
    assert msd.nn_last_error() == "inputSize % weightShape[1] != 0"
    many = torch.zeros((9, 1280), dtype=dt, device=cuda)
    out9 = torch.zeros((9, 1280), dtype=dt, device=cuda)
    assert fw(layers["time_embed_2"], _ptr(many), 9 * 1280 * es, _ptr(out9), 9 * 1280 * es, int(half), 0, 0) < 0
    for l in layers.values():
        nn.msdnn_linear_destroy(l)


def test_softmax_function_in_place_like_cross_attention(msd, nn, orc, cuda):
    x = orc.normal((8 * 64, 77), seed=400, sigma=2.0)
    xd = _dev(x, cuda)
    assert nn.msdnn_softmax(None, _ptr(xd), _ptr(xd), x.size * 4, 0, 77, 0) == 0, msd.nn_last_error()
    assert_close_f32(xd.cpu().numpy(), orc.softmax(x), what="softmax object")
    assert nn.msdnn_softmax(None, _ptr(xd), _ptr(xd), x.size * 4, 0, 76, 0) < 0
    assert msd.nn_last_error() == "element count % chunkSize != 0"


def test_ddim_sampler_object_walks_the_schedule_from_the_back(msd, nn, orc, cuda):
    """sample() with a stand-in noise model given as a callback; bit-exact against the oracle."""
    import torch
    n = 4 * 32 * 32
    x0 = orc.normal((n,), seed=500)
    noise = orc.normal((n,), seed=501)
    nd = _dev(noise, cuda)
    seen = []

    def model(x_ptr, t, e_ptr, nbytes, user):
        # e_t = 0.5 * x + (0.25 + 0.001 t) * noise, written into the sampler's e_t buffer
        seen.append(t)
        scale = float(np.float32(0.25 + 0.001 * t))
        e = cur["x"] * 0.5 + nd * scale
        msd.check(msd.load_library().msd_copy(_ptr(e), ctypes.c_void_p(e_ptr), nbytes, None))
        cur["e"] = e  # keep alive until the stream has consumed it
        return 0

    # the sampler updates its own copy of x in place; mirror it in a tensor the model can read
    steps = 25
    ts, a, ap, s1m = orc.ddim_schedule(steps)
    x = x0.copy()
    for index in range(len(ts) - 1, -1, -1):
        scale = np.float32(0.25 + 0.001 * ts[index])
        e = (np.float32(0.5) * x + scale * noise).astype(np.float32)
        x = orc.ddim_update(x, e, a[index], ap[index], s1m[index])

    xd = _dev(x0, cuda)
    out = torch.empty_like(xd)
    cur = {}

    def model_reading_sampler_memory(x_ptr, t, e_ptr, nbytes, user):
        # wrap the sampler's latent: copy it into a torch tensor first
        view = torch.empty(n, dtype=torch.float32, device=cuda)
        msd.check(msd.load_library().msd_copy(ctypes.c_void_p(x_ptr), _ptr(view), nbytes, None))
        cur["x"] = view
        return model(x_ptr, t, e_ptr, nbytes, user)

    cb = msd.MODEL_FN(model_reading_sampler_memory)
    rc = nn.msdnn_ddim_sample(None, _ptr(xd), n * 4, 0, steps, cb, None, _ptr(out))
    assert rc == 0, msd.nn_last_error()
    assert seen == [int(v) for v in ts[::-1]]  # 961, 921, ..., 1
    assert np.array_equal(xd.cpu().numpy(), x0)  # x_T untouched
    assert np.array_equal(out.cpu().numpy(), x)
    assert nn.msdnn_ddim_sample(None, _ptr(xd), n * 4, 0, 501, cb, None, _ptr(out)) < 0


def test_debug_timing_rows_like_the_reference(msd, nn, orc, cuda, tmp_path, capfd):
    """With timing on, each GroupNorm / LayerNorm forward prints the reference's CSV row
    (M/nn/GroupNorm.cpp:147-162, M/nn/LayerNorm.cpp:144-154) with one kernel per layer."""
    import torch
    np.save(tmp_path / "w.npy", np.ones(320, dtype=np.float32))
    np.save(tmp_path / "b.npy", np.zeros(320, dtype=np.float32))
    g = nn.msdnn_groupnorm_create(None, 32, 320, 1e-5, b"w.npy", b"b.npy", 2, 1)
    ln = nn.msdnn_layernorm_create(None, 320, b"w.npy", b"b.npy", 1e-5)
    assert nn.msdnn_groupnorm_init(g) == 0 and nn.msdnn_layernorm_init(ln) == 0
    x = torch.randn(2, 320, 16, 16, device=cuda)
    y = torch.empty_like(x)
    nbytes = x.numel() * 4
    capfd.readouterr()
    nn.msdnn_set_debug_timing(1)
    try:
        assert nn.msdnn_groupnorm_forward(g, _ptr(x), _ptr(y), nbytes, 0) == 0
        assert nn.msdnn_layernorm_forward(ln, _ptr(x), _ptr(y), nbytes, 0) == 0
    finally:
        nn.msdnn_set_debug_timing(0)
    err = capfd.readouterr().err
    assert "try, component, index, input size, group size, num group, weight size, workgroup size, kernel" in err
    gn_row = [l for l in err.splitlines() if l.startswith("0, GroupNorm, ")][-1].split(", ")
    assert gn_row[3:8] == [str(320 * 256), str(10 * 256), "32", "320", "64"] and gn_row[8] == "group_norm_silu"
    assert float(gn_row[9]) > 0.0
    ln_row = [l for l in err.splitlines() if l.startswith("2, LayerNorm, ")][-1].split(", ")
    assert ln_row[3:6] == [str(2 * 320 * 256), "320", "layer_norm"] and float(ln_row[6]) > 0.0
    assert nn.msdnn_groupnorm_forward(g, _ptr(x), _ptr(y), nbytes, 0) == 0
    assert "GroupNorm" not in capfd.readouterr().err  # off again
    nn.msdnn_groupnorm_destroy(g)
    nn.msdnn_layernorm_destroy(ln)


def test_layer_objects_from_cpp_against_golden_files(orc, cuda, tmp_path):
    """msd_layer_check: a C++ program that uses only the public layer headers, driven like the
    reference's in-source checks (weights and goldens as .npy under the media path)."""
    import os
    import subprocess
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    tool = os.path.join(repo, "mobile-stable-diffusion_amd", "csrc", "cli", "msd_layer_check")
    assert os.path.exists(tool), "msd_layer_check is not built: run __graft_entry__.build()"
    rnd = orc.round_to_half
    lines = []

    def save(name, a):
        np.save(tmp_path / name, np.ascontiguousarray(a, dtype=np.float32))
        return name

    # ResBlock in-norm + SiLU, fp32 and fp16 storage, batch 2
    w = orc.normal((320,), seed=601, mean=1.0, sigma=0.1)
    b = orc.normal((320,), seed=602, sigma=0.1)
    x = orc.normal((2, 320, 32, 32), seed=603, sigma=2.0)
    save("gn_w.npy", w), save("gn_b.npy", b), save("gn_x.npy", x), save("gn_x16.npy", rnd(x))
    save("gn_golden.npy", orc.groupnorm(x, w, b, 32, 1e-5, silu=True))
    save("gn_golden16.npy", rnd(orc.groupnorm(rnd(x), w, b, 32, 1e-5, silu=True)))
    lines.append("groupnorm 320 32 1e-5 2 1 f32 gn_w.npy gn_b.npy gn_x.npy gn_golden.npy")
    lines.append("groupnorm 320 32 1e-5 2 1 f16 gn_w.npy gn_b.npy gn_x16.npy gn_golden16.npy")
    # transformer LayerNorm and GEGLU
    xl = orc.normal((2 * 1024, 640), seed=604)
    wl = orc.normal((640,), seed=605, mean=1.0, sigma=0.1)
    bl = orc.normal((640,), seed=606, sigma=0.1)
    save("ln_w.npy", wl), save("ln_b.npy", bl), save("ln_x.npy", xl)
    save("ln_golden.npy", orc.layernorm(xl, wl, bl, 1e-5))
    lines.append("layernorm 640 1e-5 f32 ln_w.npy ln_b.npy ln_x.npy ln_golden.npy")
    proj = rnd(orc.normal((512, 2 * 1280), seed=607, sigma=1.5))
    save("geglu_x.npy", proj), save("geglu_golden.npy", rnd(orc.geglu(proj)))
    lines.append("geglu 320 1280 f16 geglu_x.npy geglu_golden.npy")
    # time embedding Linear with SiLU behind it, ResBlock projection with SiLU in front, no bias case
    wt = orc.normal((1280, 320), seed=608, sigma=320 ** -0.5)
    bt = orc.normal((1280,), seed=609, sigma=0.1)
    te = np.stack([orc.timestep_embedding(t) for t in (981, 1)])
    save("te_w.npy", wt), save("te_b.npy", bt), save("te_x.npy", te)
    save("te_golden.npy", orc.silu(orc.linear(te, wt, bt)))
    lines.append("linear 320 1280 0 1 f32 te_w.npy te_b.npy te_x.npy te_golden.npy")
    save("te_golden_nobias.npy", orc.linear(orc.silu(te), wt, None))
    lines.append("linear 320 1280 1 0 f32 te_w.npy - te_x.npy te_golden_nobias.npy")
    # cross-attention softmax, in place
    qk = orc.normal((8 * 256, 77), seed=610, sigma=2.0)
    save("sm_x.npy", qk), save("sm_golden.npy", orc.softmax(qk))
    lines.append("softmax 77 0 f32 sm_x.npy sm_golden.npy")
    # a golden that must fail (wrong SiLU flag) and a missing weight file: reported, not fatal
    lines.append("groupnorm 320 32 1e-5 2 0 f32 gn_w.npy gn_b.npy gn_x.npy gn_golden.npy")
    lines.append("layernorm 640 1e-5 f32 nope.npy ln_b.npy ln_x.npy ln_golden.npy")
    (tmp_path / "manifest.txt").write_text("# cases\n" + "\n".join(lines) + "\n")
    p = subprocess.run([tool, str(tmp_path), str(tmp_path / "manifest.txt")], stdout=subprocess.PIPE,
                       stderr=subprocess.PIPE, text=True, timeout=100)
    out = p.stdout.splitlines()
    verdicts = [l.split()[0] for l in out if l.startswith(("PASS", "FAIL"))]
    assert verdicts == ["PASS"] * 7 + ["FAIL", "FAIL"], p.stdout + p.stderr
    assert p.returncode == 2 and out[-1] == "7 of 9 cases passed"
    assert "max diff:" in p.stderr and "Unable to open file" in p.stderr


def test_an_earlier_hip_error_of_the_application_is_neither_reported_nor_cleared(msd, cuda):
    """Launches report the status hipLaunchKernel returns for them.  An error that an unrelated
    earlier call of the application left in the runtime's per-thread "last error" (here: a
    hipFree of a pointer nobody allocated) is not mistaken for a failed launch, and it is still
    there for the application to read afterwards."""
    import ctypes
    import torch
    path = None
    with open("/proc/self/maps") as f:
        for line in f:
            name = line.split()[-1]
            if "/libamdhip64.so" in name:
                path = name
                break
    assert path, "the HIP runtime is not mapped"
    hip = ctypes.CDLL(path)
    hip.hipFree.argtypes = [ctypes.c_void_p]
    lib = msd.load_library()
    x = torch.linspace(-4, 4, 4096, device=cuda)
    y = torch.empty_like(x)
    want = x * torch.sigmoid(x)
    torch.cuda.synchronize()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert hip.hipGetLastError() == 0
    try:
        err = hip.hipFree(ctypes.c_void_p(0x1000))          # the application's own mistake
        assert err != 0 and hip.hipPeekAtLastError() == err
        rc = lib.msd_silu(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(y.data_ptr()), x.numel(), msd.DTYPE_F32, stream)
        assert rc == 0, "an earlier error of the application came back as the launch's status"
        assert lib.msd_status(stream) == 0
        assert hip.hipPeekAtLastError() == err, "the launch cleared the application's last error"
    finally:
        hip.hipGetLastError()                               # read it, as the application would; torch checks it too
    assert torch.allclose(y, want, rtol=1e-5, atol=1e-6)
