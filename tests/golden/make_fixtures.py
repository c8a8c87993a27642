"""Writes tests/golden/fixtures.npz: small input/output vectors from library routines.

The reference ships no golden files (its .npy fixtures are git-ignored), so these
vectors come from independent textbook implementations run once on the CPU:
torch.nn.functional.{group_norm, layer_norm, silu, gelu} in float32 and the
standard sinusoidal timestep-embedding formula in float64.  They pin the CPU
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

    np.savez_compressed(OUT, **fx)
    print("wrote", OUT, os.path.getsize(OUT), "bytes,", len(fx), "arrays")


if __name__ == "__main__":
    main()
