"""CPU-side checks of the C++ layer objects (libmsd_nn.so): the NPY weight loader and the
error behaviour the reference's GroupNorm / LayerNorm / GEGLU classes have (file errors
and shape preconditions raise std::runtime_error with the reference's messages).  Nothing
here touches a GPU."""
import ctypes
import os

import numpy as np
import pytest


@pytest.fixture()
def nn(msd, tmp_path):
    lib = msd.load_nn_library()
    lib.msdnn_set_media_path(str(tmp_path).encode())
    return lib


def _load(nn, name, cap=1 << 16):
    out = (ctypes.c_float * cap)()
    n, nd = ctypes.c_size_t(0), ctypes.c_size_t(0)
    rc = nn.msdnn_npy_load(name.encode(), out, cap, ctypes.byref(n), ctypes.byref(nd))
    return rc, np.array(out[:n.value], dtype=np.float32), nd.value


def test_symbols_exported(msd):
    nn = msd.load_nn_library()
    for name in ("msdnn_groupnorm_create", "msdnn_groupnorm_init", "msdnn_groupnorm_forward",
                 "msdnn_layernorm_create", "msdnn_layernorm_forward", "msdnn_geglu_create",
                 "msdnn_geglu_forward", "msdnn_activation", "msdnn_timestep_embedding",
                 "msdnn_ddim_timesteps", "msdnn_test_buffer", "msdnn_step_run", "msdnn_npy_load"):
        assert hasattr(nn, name)


def test_npy_loader_reads_numpy_files(msd, nn, tmp_path):
    w = np.random.default_rng(1).standard_normal(320).astype(np.float32)
    np.save(tmp_path / "w.npy", w)
    rc, got, nd = _load(nn, "w.npy")
    assert rc == 0 and nd == 1 and np.array_equal(got, w)
    m = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    np.save(tmp_path / "m.npy", m)
    rc, got, nd = _load(nn, "m.npy")
    assert rc == 0 and nd == 3 and np.array_equal(got, m.reshape(-1))
    # round trip through the library's own writer, readable by numpy
    buf = (ctypes.c_float * 5)(1.5, -2.0, 0.0, 3.25, 1e-8)
    assert nn.msdnn_npy_save(str(tmp_path / "s.npy").encode(), buf, 5) == 0
    assert np.array_equal(np.load(tmp_path / "s.npy"), np.array(buf[:], dtype=np.float32))
    # version 2.0 header
    with open(tmp_path / "v2.npy", "wb") as f:
        np.lib.format.write_array(f, w, version=(2, 0))
    rc, got, _ = _load(nn, "v2.npy")
    assert rc == 0 and np.array_equal(got, w)


def test_npy_loader_errors(msd, nn, tmp_path):
    rc, _, _ = _load(nn, "missing.npy")
    assert rc < 0 and msd.nn_last_error().startswith("npy_load: Unable to open file")  # M/util.cpp:111
    np.save(tmp_path / "f8.npy", np.zeros(4, dtype=np.float64))
    rc, _, _ = _load(nn, "f8.npy")
    assert rc < 0 and "<f4" in msd.nn_last_error()
    np.save(tmp_path / "fo.npy", np.asfortranarray(np.zeros((3, 4), dtype=np.float32)))
    rc, _, _ = _load(nn, "fo.npy")
    assert rc < 0 and "Fortran" in msd.nn_last_error()
    np.save(tmp_path / "ok.npy", np.zeros(64, dtype=np.float32))
    data = (tmp_path / "ok.npy").read_bytes()
    (tmp_path / "short.npy").write_bytes(data[:-16])
    rc, _, _ = _load(nn, "short.npy")
    assert rc < 0 and msd.nn_last_error() == "nread != num_bytes"  # M/util.cpp:140
    (tmp_path / "junk.npy").write_bytes(b"not an npy file at all")
    rc, _, _ = _load(nn, "junk.npy")
    assert rc < 0 and "parse_npy_header" in msd.nn_last_error()


def test_groupnorm_init_and_forward_preconditions(msd, nn, tmp_path):
    np.save(tmp_path / "w320.npy", np.ones(320, dtype=np.float32))
    np.save(tmp_path / "b320.npy", np.zeros(320, dtype=np.float32))
    np.save(tmp_path / "b64.npy", np.zeros(64, dtype=np.float32))
    np.save(tmp_path / "w64.npy", np.ones(64, dtype=np.float32))
    g = nn.msdnn_groupnorm_create(None, 32, 320, 1e-5, b"w320.npy", b"b64.npy", 1, 0)
    assert nn.msdnn_groupnorm_init(g) < 0
    assert msd.nn_last_error() == "weight.shape[0] != bias.shape[0]"  # M/nn/GroupNorm.cpp:59-61
    nn.msdnn_groupnorm_destroy(g)
    g = nn.msdnn_groupnorm_create(None, 32, 320, 1e-5, b"w64.npy", b"b64.npy", 1, 0)
    assert nn.msdnn_groupnorm_init(g) < 0
    assert msd.nn_last_error() == "weight.shape[0] != weightSize"  # M/nn/GroupNorm.cpp:63-65
    nn.msdnn_groupnorm_destroy(g)
    g = nn.msdnn_groupnorm_create(None, 32, 320, 1e-5, b"nope.npy", b"b320.npy", 1, 0)
    assert nn.msdnn_groupnorm_init(g) < 0 and "Unable to open file" in msd.nn_last_error()
    # shape preconditions of forward (M/nn/GroupNorm.cpp:83-93), derived from the buffer size
    assert nn.msdnn_groupnorm_check(g, 320 * 64 * 64 * 4, 0) == 0
    assert nn.msdnn_groupnorm_check(g, 320 * 64 * 64 * 2, 1) == 0
    assert nn.msdnn_groupnorm_check(g, (320 * 64 + 1) * 4, 0) < 0
    assert msd.nn_last_error() == "input_size % weight->num_vals != 0"
    assert nn.msdnn_groupnorm_check(g, 320 * 3 * 4, 0) < 0  # groupSize = 30
    assert msd.nn_last_error() == "groupSize % WORK_GROUP_SIZE != 0"
    nn.msdnn_groupnorm_destroy(g)
    # batch 2: the per-sample size is what the reference calls input_size
    g = nn.msdnn_groupnorm_create(None, 32, 320, 1e-5, b"w320.npy", b"b320.npy", 2, 1)
    assert nn.msdnn_groupnorm_check(g, 2 * 320 * 64 * 2, 1) == 0
    assert nn.msdnn_groupnorm_check(g, (2 * 320 * 64 + 1) * 2, 1) < 0
    assert msd.nn_last_error() == "input_size % batch != 0"
    nn.msdnn_groupnorm_destroy(g)


def test_layernorm_and_geglu_preconditions(msd, nn, tmp_path):
    np.save(tmp_path / "w100.npy", np.ones(100, dtype=np.float32))
    np.save(tmp_path / "w320.npy", np.ones(320, dtype=np.float32))
    np.save(tmp_path / "w640.npy", np.ones(640, dtype=np.float32))
    ln = nn.msdnn_layernorm_create(None, 100, b"w100.npy", b"w100.npy", 1e-5)
    assert nn.msdnn_layernorm_init(ln) < 0
    assert msd.nn_last_error() == "weightSize % WORK_GROUP_SIZE != 0"  # M/nn/LayerNorm.cpp:61-63
    nn.msdnn_layernorm_destroy(ln)
    ln = nn.msdnn_layernorm_create(None, 320, b"w320.npy", b"w640.npy", 1e-5)
    assert nn.msdnn_layernorm_init(ln) < 0 and msd.nn_last_error() == "weightSize != biasSize"
    nn.msdnn_layernorm_destroy(ln)
    ln = nn.msdnn_layernorm_create(None, 320, b"w640.npy", b"w640.npy", 1e-5)
    assert nn.msdnn_layernorm_init(ln) < 0 and msd.nn_last_error() == "weightSize != weight->num_vals"
    assert nn.msdnn_layernorm_check(ln, 77 * 320 * 4, 0) == 0
    assert nn.msdnn_layernorm_check(ln, (77 * 320 + 5) * 4, 0) < 0
    assert msd.nn_last_error() == "input_size % weight->num_vals != 0"  # M/nn/LayerNorm.cpp:78-82
    nn.msdnn_layernorm_destroy(ln)
    ge = nn.msdnn_geglu_create(None, 320, 1280)
    r, c = ctypes.c_size_t(0), ctypes.c_size_t(0)
    nn.msdnn_geglu_weight_shape(ge, ctypes.byref(r), ctypes.byref(c))
    assert (r.value, c.value) == (2560, 320)  # Linear(in, 2*out) as in M/nn/GEGLU.cpp:33-37
    assert nn.msdnn_geglu_check(ge, 8192 * 2560 * 2, 8192 * 1280 * 2, 1) == 0
    assert nn.msdnn_geglu_check(ge, 8192 * 2561 * 2, 8192 * 1280 * 2, 1) < 0
    assert nn.msdnn_geglu_check(ge, 8192 * 2560 * 2, 8192 * 1280 * 4, 1) < 0
    nn.msdnn_geglu_destroy(ge)


def test_ddim_through_host_layer(msd, nn, orc):
    buf = (ctypes.c_int * 1000)()
    for steps in (50, 25, 30):
        n = nn.msdnn_ddim_timesteps(steps, buf, 1000)
        assert list(buf[:n]) == orc.ddim_timesteps(steps)
    assert nn.msdnn_ddim_timesteps(0, buf, 1000) < 0


def test_linear_preconditions(msd, nn, tmp_path):
    np.save(tmp_path / "w_1280x320.npy", np.zeros((1280, 320), dtype=np.float32))
    np.save(tmp_path / "b_1280.npy", np.zeros(1280, dtype=np.float32))
    np.save(tmp_path / "b_320.npy", np.zeros(320, dtype=np.float32))
    lin = nn.msdnn_linear_create(None, 320, 640, b"w_1280x320.npy", b"b_1280.npy", 0)
    assert nn.msdnn_linear_init(lin) < 0
    assert msd.nn_last_error() == "weight.num_vals != (weightShape[0] * weightShape[1])"  # M/nn/Linear.cpp:53-59
    nn.msdnn_linear_destroy(lin)
    lin = nn.msdnn_linear_create(None, 320, 1280, b"w_1280x320.npy", b"b_320.npy", 0)
    assert nn.msdnn_linear_init(lin) < 0
    assert msd.nn_last_error() == "bias.num_vals != weightShape[0]"  # M/nn/Linear.cpp:62-70
    nn.msdnn_linear_destroy(lin)
    lin = nn.msdnn_linear_create(None, 320, 1280, b"missing.npy", b"", 0)
    assert nn.msdnn_linear_init(lin) < 0 and "Unable to open file" in msd.nn_last_error()
    # forward before init
    assert nn.msdnn_linear_forward(lin, None, 0, None, 0, 0, 0, 0) < 0
    assert msd.nn_last_error() == "Linear: init() not called"
    nn.msdnn_linear_destroy(lin)


def test_ddim_make_schedule_through_sampler_object(msd, nn, orc):
    ts, a, ap, _ = orc.ddim_schedule(50)
    n = len(ts)
    t_arr = (ctypes.c_int * n)(*[int(v) for v in ts])
    ga, gp = (ctypes.c_float * n)(), (ctypes.c_float * n)()
    assert nn.msdnn_ddim_make_schedule(t_arr, n, ga, gp) == 0, msd.nn_last_error()
    assert np.array_equal(np.array(ga[:], dtype=np.float32), a)
    assert np.array_equal(np.array(gp[:], dtype=np.float32), ap)
    bad = (ctypes.c_int * 1)(1000)
    assert nn.msdnn_ddim_make_schedule(bad, 1, ga, gp) < 0  # the reference would read past its table
