"""msd_compare, the golden-file comparison tool (host only): same summary line as the
reference's util::testBuffer (M/util.cpp:167-201) and an exit status by tolerance."""
import os
import subprocess

import numpy as np
import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOOL = os.path.join(REPO, "mobile-stable-diffusion_amd", "csrc", "cli", "msd_compare")


def _run(*args):
    if not os.path.exists(TOOL):  # host-only tool: build it when a fresh checkout has none
        import importlib.util
        spec = importlib.util.spec_from_file_location(
            "msd_build", os.path.join(REPO, "mobile-stable-diffusion_amd", "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build_cli()
    p = subprocess.run([TOOL] + [str(a) for a in args], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    return p.returncode, p.stdout, p.stderr


def test_identical_and_within_tolerance(tmp_path):
    g = np.linspace(-3, 3, 1000, dtype=np.float32)
    np.save(tmp_path / "g.npy", g)
    np.save(tmp_path / "same.npy", g)
    rc, out, _ = _run(tmp_path / "same.npy", tmp_path / "g.npy")
    assert rc == 0 and "num : 0 /" in out
    r = g.copy()
    r[17] += np.float32(4e-6)
    r[500] = np.nextafter(r[500], np.float32(10))
    np.save(tmp_path / "close.npy", r)
    rc, out, _ = _run(tmp_path / "close.npy", tmp_path / "g.npy")
    assert rc == 0 and "num : 2 /" in out and "result[17]" in out
    assert "max diff: 0.0000038" in out or "max diff: 0.0000040" in out or "max diff: 0.000004" in out


def test_out_of_tolerance_size_mismatch_and_bad_files(tmp_path):
    g = np.ones((4, 8), dtype=np.float32)
    np.save(tmp_path / "g.npy", g)
    r = g.copy()
    r[2, 3] = 1.5
    np.save(tmp_path / "far.npy", r)
    rc, out, _ = _run(tmp_path / "far.npy", tmp_path / "g.npy")
    assert rc == 1 and "result[19]: 1.500000 != test[19]: 1.000000" in out and "1 of 32 elements outside" in out
    rc, _, _ = _run(tmp_path / "far.npy", tmp_path / "g.npy", "--abs", 0.6)
    assert rc == 0
    rc, _, _ = _run(tmp_path / "far.npy", tmp_path / "g.npy", "--rel", 0.6)
    assert rc == 0
    np.save(tmp_path / "short.npy", np.ones(31, dtype=np.float32))
    rc, _, err = _run(tmp_path / "short.npy", tmp_path / "g.npy")
    assert rc == 2 and "bufferSize(31) != test.num_vals(32)" in err
    rc, _, err = _run(tmp_path / "missing.npy", tmp_path / "g.npy")
    assert rc == 2 and "Unable to open file" in err
    np.save(tmp_path / "f8.npy", np.ones(32))
    rc, _, err = _run(tmp_path / "f8.npy", tmp_path / "g.npy")
    assert rc == 2 and "<f4" in err
    assert _run(tmp_path / "g.npy")[0] == 2
    nan = g.copy()
    nan[0, 0] = np.nan
    np.save(tmp_path / "nan.npy", nan)
    assert _run(tmp_path / "nan.npy", tmp_path / "g.npy")[0] == 1
