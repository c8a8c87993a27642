"""CPU-side checks of the drop-in boundary: the C-ABI library loads, exports every
symbol include/msd_hip.h declares, and its host-only entry points behave.  No
compute call is made here (there is no GPU in the CPU test environment)."""
import ctypes
import os
import re

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(REPO, "include", "msd_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(msd_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(msd):
    lib = msd.load_library()
    declared = _declared_symbols()
    assert len(declared) >= 13
    for name in declared:
        assert hasattr(lib, name), "libmsd_hip.so does not export %s" % name
    assert sorted(msd.C_ABI_SYMBOLS) == declared  # the ctypes table covers the whole header


def test_header_is_plain_c():
    text = open(os.path.join(REPO, "include", "msd_hip.h")).read()
    assert 'extern "C"' in text and "torch" not in text and "hip/hip_runtime" not in text
    # compiles as C with no HIP headers on the include path
    import subprocess
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "t.c")
        open(src, "w").write('#include "msd_hip.h"\nint main(void){return msd_ddim_timesteps(0,0,0)==-1?0:1;}\n')
        subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-c", "-I", os.path.join(REPO, "include"),
                        src, "-o", os.path.join(d, "t.o")], check=True)


def test_version_and_error_strings(msd):
    lib = msd.load_library()
    assert lib.msd_version() >= 100
    assert lib.msd_error_string(0) == b"ok"
    assert b"invalid" in lib.msd_error_string(1)


def test_ddim_timesteps_host_entry(msd, orc):
    lib = msd.load_library()
    for steps in (1, 2, 3, 7, 20, 25, 30, 50, 64, 100, 250, 333, 500, 999, 1000):
        assert msd.ddim_timesteps(steps) == orc.ddim_timesteps(steps), steps
    assert msd.ddim_timesteps(50)[-1] == 981
    assert lib.msd_ddim_timesteps(0, None, 0) == -1
    assert lib.msd_ddim_timesteps(1001, None, 0) == -1
    # cap smaller than the list: count is still returned, nothing past cap is written
    buf = (ctypes.c_int * 4)(-7, -7, -7, -7)
    assert lib.msd_ddim_timesteps(50, buf, 3) == 50
    assert list(buf) == [1, 21, 41, -7]
    with pytest.raises(msd.MsdError):
        msd.ddim_timesteps(0)


def test_argument_validation_needs_no_gpu(msd):
    lib = msd.load_library()
    # rejected before any HIP call
    assert lib.msd_groupnorm(None, None, None, None, 1, 30, 16, 32, 1e-5, 0, 0, None) == 1
    assert lib.msd_groupnorm(None, None, None, None, 1, 32, 16, 0, 1e-5, 0, 0, None) == 1
    assert lib.msd_layernorm(None, None, None, None, 4, 64, 1e-5, 0, None) == 1
    assert lib.msd_geglu(None, None, 4, 64, 0, None) == 1
    assert lib.msd_silu(None, None, 4, 0, None) == 1
    assert lib.msd_timestep_embedding(None, None, 2, 321, 10000.0, 0, None) == 1
    assert lib.msd_set_tuning(0, 3) == 1      # split must be a power of two
    assert lib.msd_set_tuning(1, 100) == 1    # threads must be a multiple of 64
    assert lib.msd_set_tuning(2, 12) == 1 and lib.msd_set_tuning(4, 3) == 1 and lib.msd_set_tuning(99, 1) == 1
    assert lib.msd_set_tuning(6, 48) == 1     # softmax rows per workgroup: 16, 32 or 64
    assert lib.msd_set_tuning(9, 0) == 1      # no such knob
    assert lib.msd_set_tuning(8, 3) == 1 and lib.msd_set_tuning(8, 32) == 1   # writers: a power of two up to 16
    for knob in range(9):
        assert lib.msd_set_tuning(knob, 0) == 0
    # GEGLU rows of input and output have different strides: any overlap is refused
    # (addresses are never dereferenced: the check comes before the launch)
    base = 1 << 20
    rows, inner = 4, 64  # fp16: proj 4 * 128 * 2 = 1024 bytes, out 512 bytes
    p = ctypes.c_void_p
    assert lib.msd_geglu(p(base), p(base), rows, inner, 1, None) == 1            # in place
    assert lib.msd_geglu(p(base), p(base + 1008), rows, inner, 1, None) == 1     # out starts inside proj
    assert lib.msd_geglu(p(base + 496), p(base), rows, inner, 1, None) == 1      # proj starts inside out
    # the entry point with the fixed scratch refuses more units than that scratch holds,
    # before it touches a device
    assert lib.msd_groupnorm_noalloc(p(base), p(base), p(base), p(base), 33, 64, 16, 32, 1e-5, 0, 0, None) == -2
    assert lib.msd_groupnorm_noalloc(p(base), p(base), p(base), p(base), 2, 2050, 16, 2050, 1e-5, 0, 0, None) == -2
    assert b"1024" in lib.msd_error_string(-2)
    assert lib.msd_gn_fallbacks(None, None, 0) == 1
    # the neighbours of the path
    assert lib.msd_linear_rows(None, None, None, None, 9, 4, 8, 0, 0, 0, None) == 1   # more than 8 rows
    assert lib.msd_linear_rows(None, None, None, None, 2, 4, 8, 0, 0, 0, None) == 1   # null pointers
    assert lib.msd_linear_rows(None, None, None, None, 2, 4, 8, 3, 0, 0, None) == 1   # unknown activation
    assert lib.msd_linear_rows_grouped(None, None, None, None, None, 2, 2, 8, 0, 0, 0, None) == 1  # null tables
    assert lib.msd_linear_rows_grouped(None, None, None, None, None, 0, 2, 8, 0, 0, 0, None) == 0  # nothing to do
    assert lib.msd_softmax(None, None, 4, 77, 0, 0, None) == 1
    assert lib.msd_softmax(None, None, 0, 77, 0, 0, None) == 0                        # empty: nothing to do
    assert lib.msd_ddim_update(None, None, None, 16, 0.5, 0.5, 0.7, 0, None) == 1
    one = ctypes.c_void_p(16)  # never dereferenced: the coefficients are rejected first
    assert lib.msd_ddim_update(one, one, one, 16, 0.0, 0.5, 0.7, 0, None) == 1        # a_t must be > 0
    assert lib.msd_ddim_update(one, one, one, 16, 0.5, 1.5, 0.7, 0, None) == 1        # a_prev in [0, 1]
    assert lib.msd_alphas_cumprod(None) == 1
    assert lib.msd_ddim_schedule(50, None, None, None, None, 0) == 50
    assert lib.msd_ddim_schedule(501, None, None, None, None, 0) == -2


def test_missing_library_fails_loudly(msd):
    with pytest.raises(msd.MsdError):
        msd.load_library(os.path.join(REPO, "does_not_exist.so"))
