"""Pins the oracle's restatements of the path's neighbours: the embedding Linear,
the row softmax, the DDIM alpha schedule and the DDIM update.

Same rules as test_oracle_pinning.py: library fixtures (torch, float32 / float64),
float64 brute force, and closed forms chosen so that a transposed operand, a dropped
bias, a wrong shift of alphas_prev or a swapped a_t / a_prev fails one of them.
"""
import math

import numpy as np
import pytest

from tolerances import assert_close_f32


# ----------------------------------------------------------------- Linear
@pytest.mark.parametrize("name", ["lin_a", "lin_b", "lin_c"])
def test_linear_matches_library_fixture(orc, golden, name):
    x, w = golden[name + "_x"], golden[name + "_w"]
    b = golden[name + "_b"] if name + "_b" in golden.files else None
    assert_close_f32(orc.linear(x, w, b), golden[name + "_y"], 1e-5, name)
    assert_close_f32(orc.linear(orc.silu(x), w, b), golden[name + "_y_silu_in"], 1e-5, name + " silu in")
    assert_close_f32(orc.silu(orc.linear(x, w, b)), golden[name + "_y_silu_out"], 1e-5, name + " silu out")


def test_linear_matches_float64_and_numpy(orc):
    x = orc.normal((3, 200), seed=71)
    w = orc.normal((11, 200), seed=72, sigma=0.07)
    b = orc.normal((11,), seed=73)
    ref = x.astype(np.float64) @ w.astype(np.float64).T + b.astype(np.float64)
    np.testing.assert_allclose(orc.linear64(x, w, b), ref, rtol=0, atol=1e-12)
    assert_close_f32(orc.linear(x, w, b), ref, 2e-6, "linear vs f64")
    assert_close_f32(orc.linear(x, w, None), ref - b, 2e-6, "linear without bias")


def test_linear_one_hot_rows_select_single_weights(orc):
    # x = e_k picks column k of W exactly: a transposed or mis-strided weight index fails
    n, k = 7, 12
    w = orc.normal((n, k), seed=74)
    x = np.eye(k, dtype=np.float32)[[0, 5, 11]]
    y = orc.linear(x, w, None)
    assert np.array_equal(y, w[:, [0, 5, 11]].T)


# ----------------------------------------------------------------- softmax
@pytest.mark.parametrize("name", ["sm_a", "sm_b", "sm_c"])
def test_softmax_matches_library_fixture(orc, golden, name):
    x = golden[name + "_x"]
    y = orc.softmax(x)
    np.testing.assert_allclose(y, golden[name + "_y"], rtol=2e-6, atol=1e-9)
    np.testing.assert_allclose(y.astype(np.float64).sum(axis=-1), 1.0, atol=2e-6)


def test_softmax_matches_float64_and_is_shift_invariant(orc):
    x = orc.normal((5, 333), seed=81, sigma=2.5)
    ref = orc.softmax64(x)
    np.testing.assert_allclose(orc.softmax(x), ref, rtol=3e-6, atol=1e-10)
    np.testing.assert_allclose(orc.softmax64(x + np.float32(4.0)), ref, rtol=1e-6, atol=1e-12)


@pytest.mark.parametrize("local_size", [1, 2, 5, 7, 64, 100])
def test_softmax_tree_handles_any_workgroup_size(orc, local_size):
    # the odd-size bookkeeping of the reduction tree must still add every partial sum once
    x = orc.normal((3, 150), seed=82)
    np.testing.assert_allclose(orc.softmax(x, local_size), orc.softmax64(x), rtol=3e-6, atol=1e-10)


def test_softmax_has_no_max_subtraction(orc):
    # exp(89) overflows float32: the reference form yields inf/inf = nan there, and
    # zero for the finite neighbours; a restatement that subtracts the maximum would not
    x = np.array([[0.0, 89.0, 1.0]], dtype=np.float32)
    with np.errstate(all="ignore"):
        y = orc.softmax(x)
    assert np.isnan(y[0, 1]) and y[0, 0] == 0.0 and y[0, 2] == 0.0


# ----------------------------------------------------------------- DDIM schedule
def test_alphas_cumprod_matches_ldm_schedule(orc, golden):
    acp = orc.alphas_cumprod()
    ref = golden["ddim_alphas_cumprod_f64"]
    assert acp.dtype == np.float32 and acp.shape == (1000,)
    assert np.array_equal(acp, ref.astype(np.float32))  # float64 product rounded once
    # published end points of the Stable Diffusion v1 schedule
    assert abs(float(acp[0]) - 0.99915) < 1e-7
    assert abs(float(acp[999]) - 0.0046601) < 1e-7
    assert np.all(np.diff(acp.astype(np.float64)) < 0)


@pytest.mark.parametrize("steps", [50, 25, 30, 7, 1])
def test_ddim_schedule_gathers_and_shifts(orc, golden, steps):
    ts, a, ap, s1m = orc.ddim_schedule(steps)
    assert ts.tolist() == orc.ddim_timesteps(steps)
    acp = golden["ddim_alphas_cumprod_f64"].astype(np.float32)
    assert np.array_equal(a, acp[ts])
    assert ap[0] == acp[0] and np.array_equal(ap[1:], a[:-1])  # previous entry, first = cumprod[0]
    assert np.array_equal(s1m, np.sqrt(np.float32(1.0) - a))


def test_ddim_schedule_rejects_what_the_reference_cannot_index(orc):
    with pytest.raises(ValueError):
        orc.ddim_schedule(0)
    with pytest.raises(ValueError):
        orc.ddim_schedule(1001)
    with pytest.raises(ValueError):
        orc.ddim_schedule(1000)  # stride 1: the list ends at 1000, one past the table
    with pytest.raises(ValueError):
        orc.ddim_schedule(501)
    assert len(orc.ddim_schedule(500)[0]) == 500  # stride 2: 1, 3, ..., 999


# ----------------------------------------------------------------- DDIM update
def test_ddim_update_matches_float64_fixture(orc, golden):
    x, e = golden["ddim_x"], golden["ddim_e"]
    a_t, a_prev = float(golden["ddim_a_t"]), float(golden["ddim_a_prev"])
    a_t32, a_prev32 = np.float32(a_t), np.float32(a_prev)
    got = orc.ddim_update(x, e, a_t32, a_prev32, np.sqrt(np.float32(1.0) - a_t32))
    assert_close_f32(got, golden["ddim_x_prev_f64"], 2e-6, "ddim update vs LDM f64")
    np.testing.assert_allclose(orc.ddim_update64(x, e, a_t, a_prev), golden["ddim_x_prev_f64"],
                               rtol=0, atol=1e-12)


def test_ddim_update_special_cases(orc):
    x = orc.normal((1024,), seed=91)
    e = orc.normal((1024,), seed=92)
    a_t, a_prev = np.float32(0.36), np.float32(0.81)
    s1m = np.sqrt(np.float32(1.0) - a_t)
    # e_t = 0: x_prev = sqrt(a_prev) * (x / sqrt(a_t)); swapping a_t and a_prev fails this
    got = orc.ddim_update(x, np.zeros_like(x), a_t, a_prev, s1m)
    want = np.sqrt(a_prev) * (x / np.sqrt(a_t))
    assert np.array_equal(got, want.astype(np.float32))
    # a_prev = a_t: the step is the identity up to rounding; a wrong sign on either e_t term fails
    same = orc.ddim_update(x, e, a_t, a_t, s1m)
    assert_close_f32(same, x, 1e-6, "ddim identity step")
    # x = 0, a_t = a_prev -> exactly... dir - dir: bounded by rounding of the two products
    z = orc.ddim_update(np.zeros_like(x), e, a_t, a_t, s1m)
    assert np.abs(z).max() < 1e-6
