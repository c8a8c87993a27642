"""Writes tests/golden/fixtures.npz: small input/output vectors from library routines.

The reference ships no golden files (its .npy fixtures are git-ignored), so these
vectors come from independent textbook implementations run once on the CPU:
torch.nn.functional.{group_norm, layer_norm, silu, gelu, linear}, torch.softmax in
float32, the standard sinusoidal timestep-embedding formula and the LDM beta
schedule / DDIM step in float64.  They pin the CPU
oracle (tests/test_oracle_pinning.py) and are re-checked against the HIP
kernels (tests/test_gpu_parity.py).  Inputs come from numpy's PCG64 with fixed
seeds, so re-running this script reproduces the file bit for bit on the same
torch build.

    python tests/golden/make_fixtures.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fixtures.npz")


def main():
    torch.manual_seed(0)
    torch.set_num_threads(1)
    rng = np.random.Generator(np.random.PCG64(20231207))
    fx = {}

    # GroupNorm(32) cases: (name, batch, C, H, W, eps, sigma, offset)
    for name, b, c, h, w, eps, sigma, off in [
        ("gn_a", 1, 64, 8, 8, 1e-5, 1.0, 0.0),
        ("gn_b", 2, 320, 8, 8, 1e-5, 2.0, 0.5),
        ("gn_c", 1, 128, 4, 8, 1e-6, 0.5, -3.0),
    ]:
        x = (rng.standard_normal((b, c, h, w)) * sigma + off).astype(np.float32)
        g = (1.0 + 0.1 * rng.standard_normal(c)).astype(np.float32)
        be = (0.1 * rng.standard_normal(c)).astype(np.float32)
        y = F.group_norm(torch.from_numpy(x), 32, torch.from_numpy(g), torch.from_numpy(be), eps)
        fx[name + "_x"], fx[name + "_gamma"], fx[name + "_beta"] = x, g, be
        fx[name + "_eps"] = np.float32(eps)
        fx[name + "_y"] = y.numpy()
        fx[name + "_y_silu"] = F.silu(y).numpy()

    # LayerNorm cases
    for name, rows, dim, eps in [("ln_a", 16, 320, 1e-5), ("ln_b", 7, 768, 1e-5),
                                 ("ln_c", 5, 1024, 1e-5), ("ln_d", 3, 1280, 1e-5)]:
        x = rng.standard_normal((rows, dim)).astype(np.float32)
        x[rng.random((rows, dim)) < 0.01] = 20.0
        g = (1.0 + 0.1 * rng.standard_normal(dim)).astype(np.float32)
        be = (0.1 * rng.standard_normal(dim)).astype(np.float32)
        y = F.layer_norm(torch.from_numpy(x), (dim,), torch.from_numpy(g), torch.from_numpy(be), eps)
        fx[name + "_x"], fx[name + "_gamma"], fx[name + "_beta"] = x, g, be
        fx[name + "_eps"] = np.float32(eps)
        fx[name + "_y"] = y.numpy()

    # activations: a sweep plus random values
    xs = np.concatenate([np.linspace(-12.0, 12.0, 2049), rng.standard_normal(2047) * 3.0,
                         np.array([0.0, -0.0, 1.0, -1.0])]).astype(np.float32)
    tx = torch.from_numpy(xs)
    fx["act_x"] = xs
    fx["act_silu"] = F.silu(tx).numpy()
    fx["act_gelu"] = F.gelu(tx).numpy()  # erf form
    fx["act_quick_gelu"] = (tx * torch.sigmoid(1.702 * tx)).numpy()
    fx["act_gelu_f64"] = F.gelu(tx.double()).numpy()

    # GEGLU as written by diffusers / LDM: value, gate = proj.chunk(2, -1); value * gelu(gate)
    proj = rng.standard_normal((8, 2 * 64)).astype(np.float32) * 1.5
    value, gate = torch.from_numpy(proj).chunk(2, dim=-1)
    fx["geglu_proj"] = proj
    fx["geglu_y"] = (value * F.gelu(gate)).numpy()

    # sinusoidal timestep embedding (LDM timestep_embedding), float64 ground truth
    ts = np.array([0, 1, 2, 21, 500, 961, 981, 999], dtype=np.int64)
    half = 160
    freqs = np.exp(-np.log(10000.0) * np.arange(half, dtype=np.float64) / half)
    args = ts[:, None].astype(np.float64) * freqs[None, :]
    fx["temb_t"] = ts
    fx["temb_f64"] = np.concatenate([np.cos(args), np.sin(args)], axis=1)

    # ---- neighbours of the path (drawn after everything above, so the earlier arrays keep
    # their values): Linear, row softmax, the LDM "linear" beta schedule and one DDIM step
    for name, m, n, k, with_bias in [("lin_a", 2, 48, 320, True), ("lin_b", 2, 40, 1280, True),
                                     ("lin_c", 3, 17, 96, False)]:
        x = rng.standard_normal((m, k)).astype(np.float32)
        w = (rng.standard_normal((n, k)) / np.sqrt(k)).astype(np.float32)
        b = (0.1 * rng.standard_normal(n)).astype(np.float32) if with_bias else None
        tb = torch.from_numpy(b) if with_bias else None
        fx[name + "_x"], fx[name + "_w"] = x, w
        if with_bias:
            fx[name + "_b"] = b
        fx[name + "_y"] = F.linear(torch.from_numpy(x), torch.from_numpy(w), tb).numpy()
        fx[name + "_y_silu_in"] = F.linear(F.silu(torch.from_numpy(x)), torch.from_numpy(w), tb).numpy()
        fx[name + "_y_silu_out"] = F.silu(F.linear(torch.from_numpy(x), torch.from_numpy(w), tb)).numpy()

    for name, rows, cols, sigma in [("sm_a", 6, 77, 2.0), ("sm_b", 4, 256, 3.0), ("sm_c", 3, 1000, 1.0)]:
        x = (rng.standard_normal((rows, cols)) * sigma).astype(np.float32)
        fx[name + "_x"] = x
        fx[name + "_y"] = torch.softmax(torch.from_numpy(x), dim=-1).numpy()

    # LDM make_beta_schedule("linear", 1000, 0.00085, 0.0120) and its running product, float64
    betas = torch.linspace(0.00085 ** 0.5, 0.0120 ** 0.5, 1000, dtype=torch.float64) ** 2
    acp = torch.cumprod(1.0 - betas, dim=0)
    fx["ddim_alphas_cumprod_f64"] = acp.numpy()
    # one DDIM step (eta 0) of LDM's p_sample_ddim in float64 at step index 30 of 50
    ddim_ts = np.arange(0, 1000, 1000 // 50) + 1
    a_t, a_prev = float(acp[ddim_ts[30]]), float(acp[ddim_ts[29]])
    x = rng.standard_normal(4 * 16 * 16).astype(np.float32)
    e = rng.standard_normal(4 * 16 * 16).astype(np.float32)
    xd, ed = torch.from_numpy(x).double(), torch.from_numpy(e).double()
    pred_x0 = (xd - (1.0 - a_t) ** 0.5 * ed) / a_t ** 0.5
    fx["ddim_x"], fx["ddim_e"] = x, e
    fx["ddim_a_t"], fx["ddim_a_prev"] = np.float64(a_t), np.float64(a_prev)
    fx["ddim_x_prev_f64"] = (a_prev ** 0.5 * pred_x0 + (1.0 - a_prev) ** 0.5 * ed).numpy()

    np.savez_compressed(OUT, **fx)
    print("wrote", OUT, os.path.getsize(OUT), "bytes,", len(fx), "arrays")


if __name__ == "__main__":
    main()
