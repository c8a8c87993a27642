"""Pins the CPU oracle before anything is compared against it.

The reference holds no golden vectors for this path (its fixtures are
git-ignored), so each oracle function is checked against (1) committed vectors
from independent library routines (tests/golden/fixtures.npz), (2) float64
brute force, and (3) what the mathematics fixes: closed forms, invariants and
special cases chosen so that a dropped term, a wrong index or a swapped operand
fails at least one of them.
"""
import math

import numpy as np
import pytest

from tolerances import assert_close_f32

# The reference's own recorded agreement with PyTorch fp32 on its phone GPU is
# 9.5e-7 .. 7.3e-6 for GroupNorm and up to 5.4e-6 for the UNet LayerNorms
# (comments at M/nn/ResBlock.cpp:129-133, M/nn/BasicTransformerBlock.cpp:119-161);
# the restatement must be at least that close to the same library routines.
LIB_TOL = 1e-5


# ----------------------------------------------------------------- GroupNorm
@pytest.mark.parametrize("name", ["gn_a", "gn_b", "gn_c"])
def test_groupnorm_matches_library_fixture(orc, golden, name):
    x, g, b = golden[name + "_x"], golden[name + "_gamma"], golden[name + "_beta"]
    eps = float(golden[name + "_eps"])
    assert_close_f32(orc.groupnorm(x, g, b, 32, eps, silu=False), golden[name + "_y"], LIB_TOL, name)
    assert_close_f32(orc.groupnorm(x, g, b, 32, eps, silu=True), golden[name + "_y_silu"], LIB_TOL,
                     name + "+silu")


def test_groupnorm_matches_float64_bruteforce(orc):
    x = orc.normal((2, 96, 4, 16), seed=11, mean=0.3, sigma=2.0)  # 3 channels/group, G = 192
    g = orc.normal((96,), seed=12, mean=1.0, sigma=0.1)
    b = orc.normal((96,), seed=13, mean=0.0, sigma=0.1)
    for silu in (False, True):
        assert_close_f32(orc.groupnorm(x, g, b, 32, 1e-5, silu), orc.groupnorm64(x, g, b, 32, 1e-5, silu),
                         2e-6, "gn vs f64")


def test_groupnorm_constant_input_gives_beta_exactly(orc):
    # x - mean == 0 exactly, so y == fma(0, w, b) == b: catches a wrong channel index
    x = np.full((1, 64, 8, 8), 3.25, dtype=np.float32)
    g = orc.normal((64,), seed=1, mean=1.0, sigma=0.1)
    b = orc.normal((64,), seed=2)
    y = orc.groupnorm(x, g, b, 32, 1e-5)
    assert np.array_equal(y, np.broadcast_to(b[None, :, None, None], y.shape))


def test_groupnorm_unit_statistics_and_biased_variance(orc):
    # gamma=1, beta=0: each group has mean 0 and biased variance var/(var+eps).
    x = orc.normal((1, 64, 8, 8), seed=5, mean=1.0, sigma=0.01)  # small var: eps matters
    one, zero = np.ones(64, np.float32), np.zeros(64, np.float32)
    eps = 1e-5
    y = orc.groupnorm(x, one, zero, 32, eps).astype(np.float64).reshape(32, -1)
    xv = x.astype(np.float64).reshape(32, -1).var(axis=1)  # biased (ddof=0)
    assert np.abs(y.mean(axis=1)).max() < 1e-4  # fp32 mean of values near 1, scaled by 1/std ~ 1e2
    np.testing.assert_allclose(y.var(axis=1), xv / (xv + eps), rtol=2e-4)
    # an unbiased (N-1) variance would be off by 1/128 = 7.8e-3 relative: excluded by rtol


def test_groupnorm_groups_are_independent_per_sample(orc):
    # batch handling: sample 1 must not see sample 0's statistics
    x = orc.normal((2, 64, 8, 8), seed=21, sigma=1.0)
    x[1] = x[1] * 5.0 + 7.0
    g = np.ones(64, np.float32)
    b = np.zeros(64, np.float32)
    both = orc.groupnorm(x, g, b, 32)
    assert np.array_equal(both[0], orc.groupnorm(x[:1], g, b, 32)[0])
    assert np.array_equal(both[1], orc.groupnorm(x[1:], g, b, 32)[0])


def test_groupnorm_reference_preconditions(orc):
    g = np.ones(32, np.float32)
    with pytest.raises(ValueError):  # groupSize % 64 != 0 (M/nn/GroupNorm.cpp:89-93)
        orc.groupnorm(np.zeros((1, 32, 3, 3), np.float32), g, g, 32)


def test_reduction_kernels_individually(orc):
    # 3 workgroups x (64 lanes x R=4): mean and biased variance of each 256-slab
    x = orc.normal((3, 256), seed=31, mean=-2.0, sigma=3.0)
    mean = np.empty(3, np.float32)
    var = np.empty(3, np.float32)
    orc.lib().orc_local_reduction_mean(x.reshape(-1), mean, 3, 4)
    orc.lib().orc_local_reduction_variance(x.reshape(-1), mean, var, 3, 4)
    np.testing.assert_allclose(mean, x.astype(np.float64).mean(axis=1), rtol=1e-6)
    np.testing.assert_allclose(var, x.astype(np.float64).var(axis=1), rtol=1e-5)
    # powers of two are summed exactly in any order: the tree must give the exact mean
    p = np.tile(np.array([1.0, 2.0, 4.0, 8.0], np.float32), 64)
    orc.lib().orc_local_reduction_mean(p, mean[:1], 1, 4)
    assert mean[0] == np.float32(3.75)


# ----------------------------------------------------------------- LayerNorm
@pytest.mark.parametrize("name", ["ln_a", "ln_b", "ln_c", "ln_d"])
def test_layernorm_matches_library_fixture(orc, golden, name):
    x, g, b = golden[name + "_x"], golden[name + "_gamma"], golden[name + "_beta"]
    assert_close_f32(orc.layernorm(x, g, b, float(golden[name + "_eps"])), golden[name + "_y"], LIB_TOL, name)


def test_layernorm_float64_and_column_indexing(orc):
    x = orc.normal((9, 640), seed=41, sigma=1.5)
    orc.add_outliers(x, seed=42)
    g = orc.normal((640,), seed=43, mean=1.0, sigma=0.2)
    b = orc.normal((640,), seed=44)
    assert_close_f32(orc.layernorm(x, g, b), orc.layernorm64(x, g, b), 3e-6, "ln vs f64")
    # constant rows: output is beta by column (catches chunkID / chunkGroupID swapped)
    c = np.repeat(np.arange(9, dtype=np.float32)[:, None], 640, axis=1)
    assert np.array_equal(orc.layernorm(c, g, b), np.broadcast_to(b, (9, 640)))
    with pytest.raises(ValueError):  # dim % 64 != 0 (M/nn/LayerNorm.cpp:61)
        orc.layernorm(np.zeros((2, 100), np.float32), np.ones(100, np.float32), np.ones(100, np.float32))


# ----------------------------------------------------------------- activations
def test_activations_match_library_fixture(orc, golden):
    x = golden["act_x"]
    assert_close_f32(orc.silu(x), golden["act_silu"], 2e-6, "silu")
    assert_close_f32(orc.gelu(x), golden["act_gelu"], 2e-6, "gelu")
    assert_close_f32(orc.gelu(x), golden["act_gelu_f64"], 2e-6, "gelu f64")
    assert_close_f32(orc.quick_gelu(x), golden["act_quick_gelu"], 2e-6, "quick_gelu")


def test_activation_closed_forms(orc):
    x = np.array([0.0, 1.0, -1.0, 30.0, -30.0, 0.5], np.float32)
    s = orc.silu(x)
    assert s[0] == 0.0
    assert abs(s[1] - 0.7310585786300049) < 1e-7
    assert abs(s[2] + 0.2689414213699951) < 1e-7
    assert s[3] == np.float32(30.0) and abs(s[4]) < 1e-11
    ge = orc.gelu(x)
    assert ge[0] == 0.0
    assert abs(ge[1] - 0.8413447460685429) < 1e-7
    assert abs(ge[2] + 0.15865525393145707) < 1e-7
    # gelu(x) - gelu(-x) == x (Phi(x) + Phi(-x) == 1): fails on a sign or 0.5 slip
    xs = np.linspace(-6, 6, 241).astype(np.float32)
    np.testing.assert_allclose(orc.gelu(xs) - orc.gelu(-xs), xs, atol=1e-6)
    # the erf form differs from the tanh approximation by up to ~4.7e-4: must be erf
    tanh_form = 0.5 * xs * (1 + np.tanh(math.sqrt(2 / math.pi) * (xs + 0.044715 * xs ** 3)))
    assert np.abs(orc.gelu(xs) - tanh_form).max() > 1e-4
    q = orc.quick_gelu(x)
    assert abs(q[1] - 1.0 / (1.0 + math.exp(-1.702))) < 1e-7
    assert_close_f32(orc.silu(xs), orc.silu64(xs), 1e-6)
    assert_close_f32(orc.quick_gelu(xs), orc.quick_gelu64(xs), 1e-6)


def test_geglu_half_order_and_fixture(orc, golden):
    assert_close_f32(orc.geglu(golden["geglu_proj"]), golden["geglu_y"], 2e-6, "geglu")
    # value is the FIRST half, gate the SECOND (K/geglu.cl:7-8,24)
    x = np.linspace(-4, 4, 64).astype(np.float32)
    gate_second = np.concatenate([np.ones(64, np.float32), x])[None, :]
    np.testing.assert_array_equal(orc.geglu(gate_second)[0], orc.gelu(x))
    value_first = np.concatenate([x, np.full(64, 40.0, np.float32)])[None, :]  # gelu(40) == 40
    np.testing.assert_array_equal(orc.geglu(value_first)[0], x * np.float32(40.0))
    # row stride is 2*inner (a wrong stride mixes rows)
    ab = orc.normal((5, 256), seed=51)
    got = orc.geglu(ab)
    for r in range(5):
        np.testing.assert_array_equal(got[r], orc.geglu(ab[r:r + 1])[0])
    assert_close_f32(got, orc.geglu64(ab), 2e-6)


def test_add_kernels_are_exact(orc):
    a = orc.normal((2, 6, 5, 7), seed=81, sigma=3.0)
    b = orc.normal((2, 6, 5, 7), seed=82)
    assert np.array_equal(orc.elemwise_add(a, b), a + b)
    chunk = orc.normal((2, 6), seed=83)  # one value per (sample, channel), broadcast over H*W
    assert np.array_equal(orc.chunkwise_add(a, chunk, 35), a + chunk[:, :, None, None])
    t = orc.normal((3, 5, 7), seed=84)
    assert np.array_equal(orc.permute_0_2_1(t), t.transpose(0, 2, 1))


# ----------------------------------------------------------------- timestep embedding
def test_timestep_embedding_closed_forms(orc, golden):
    e0 = orc.timestep_embedding(0)
    assert np.array_equal(e0[:160], np.ones(160, np.float32))  # cos first ...
    assert np.array_equal(e0[160:], np.zeros(160, np.float32))  # ... then sin
    for t in (1, 7, 981):
        e = orc.timestep_embedding(t)
        assert abs(e[0] - math.cos(t)) < 1e-6 and abs(e[160] - math.sin(t)) < 1e-6  # f_0 == 1
        np.testing.assert_allclose(e[:160] ** 2 + e[160:] ** 2, 1.0, atol=3e-7)
    f = orc.timestep_freqs()
    assert f[0] == 1.0 and np.all(np.diff(f) < 0)
    assert abs(f[159] - 10000.0 ** (-159.0 / 160.0)) < 1e-9  # divides by half, not half-1
    # float64 ground truth: the float32 loop is within |t| * ulp(freq) of it
    for k, t in enumerate(golden["temb_t"]):
        e = orc.timestep_embedding(int(t))
        assert np.abs(e - golden["temb_f64"][k]).max() <= 1e-7 + abs(int(t)) * 1.2e-7
        assert np.abs(e - orc.timestep_embedding64(int(t))).max() <= 1e-7 + abs(int(t)) * 1.2e-7


def test_timestep_embedding_other_dims(orc):
    e = orc.timestep_embedding(13, dim=64, max_period=100.0)
    i = np.arange(32)
    ref = 13.0 * np.exp(-math.log(100.0) * i / 32.0)
    np.testing.assert_allclose(e[:32], np.cos(ref), atol=2e-6)
    np.testing.assert_allclose(e[32:], np.sin(ref), atol=2e-6)


# ----------------------------------------------------------------- DDIM integer list
def test_ddim_timesteps(orc):
    t50 = orc.ddim_timesteps(50)
    assert t50 == [1 + 20 * k for k in range(50)]
    assert t50[-1] == 981  # the literal the shipped app passes as its first step (native-lib.cpp:240)
    assert orc.ddim_timesteps(25) == [1 + 40 * k for k in range(25)]
    t30 = orc.ddim_timesteps(30)  # 1000 // 30 == 33 -> 31 entries, 1 .. 991
    assert len(t30) == 31 and t30[0] == 1 and t30[-1] == 991 and t30[1] - t30[0] == 33
    assert orc.ddim_timesteps(1000) == list(range(1, 1001))
    assert orc.ddim_timesteps(1) == [1]
    assert orc.ddim_timesteps(999) == list(range(1, 1001))  # c == 1
    with pytest.raises(ValueError):
        orc.ddim_timesteps(0)


# ----------------------------------------------------------------- fp16 emulation + data
def test_half_rounding_matches_numpy(orc):
    x = np.concatenate([
        orc.normal((20000,), seed=61, sigma=3.0),
        orc.normal((5000,), seed=62, sigma=1e-5),  # subnormal halves
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e6, -1e6, 5.96e-8, 2.98e-8, 2.9e-8,
                  6.1035e-5, 1.0009765625, 1.00048828125, 1.00146484375], np.float32),
    ])
    with np.errstate(over="ignore"):
        ref = x.astype(np.float16)
    assert np.array_equal(orc.to_half_bits(x), ref.view(np.uint16))
    assert np.array_equal(orc.round_to_half(x), ref.astype(np.float32))
    assert np.array_equal(orc.from_half_bits(ref.view(np.uint16)), ref.astype(np.float32))
    allbits = np.arange(0x7C00, dtype=np.uint16)  # every finite non-negative half
    assert np.array_equal(orc.to_half_bits(orc.from_half_bits(allbits)), allbits)


def test_generator_is_deterministic_and_normal(orc):
    a = orc.normal((200001,), seed=7, mean=1.0, sigma=2.0)
    assert np.array_equal(a, orc.normal((200001,), seed=7, mean=1.0, sigma=2.0))
    assert not np.array_equal(a, orc.normal((200001,), seed=8, mean=1.0, sigma=2.0))
    assert abs(a.mean() - 1.0) < 0.02 and abs(a.std() - 2.0) < 0.02
    o = orc.add_outliers(np.zeros(100000, np.float32), seed=3)
    frac = (o != 0).mean()
    assert 0.007 < frac < 0.013 and set(np.unique(o)) == {-20.0, 0.0, 20.0}
    t = orc.uniform_int(5000, 9, 0, 999)
    assert t.min() >= 0 and t.max() <= 999 and len(np.unique(t)) > 900


def test_results_do_not_depend_on_thread_count(orc):
    x = orc.normal((2, 320, 16, 16), seed=71, sigma=2.0)
    g = orc.normal((320,), seed=72, mean=1.0, sigma=0.1)
    b = orc.normal((320,), seed=73, sigma=0.1)
    n = orc.max_threads()
    orc.set_threads(1)
    one = orc.groupnorm(x, g, b, 32, silu=True)
    orc.set_threads(n)
    assert np.array_equal(one, orc.groupnorm(x, g, b, 32, silu=True))
