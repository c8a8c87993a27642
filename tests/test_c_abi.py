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
    assert lib.msd_set_tuning(12, 0) == 1     # no such knob
    assert lib.msd_set_tuning(8, 3) == 1 and lib.msd_set_tuning(8, 32) == 1   # writers: a power of two up to 16
    assert lib.msd_set_tuning(9, 5000) == 1 and lib.msd_set_tuning(10, 65) == 1 and lib.msd_set_tuning(11, 2) == 1
    for knob in range(12):
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


def test_shifted_overlaps_are_refused_before_any_launch(msd):
    """An output that may alias an input must be that input exactly or lie apart from it; an
    output that must not overlap an input may not share a byte with it.  The addresses are
    never dereferenced: every call below returns before anything is launched."""
    lib = msd.load_library()
    p = ctypes.c_void_p
    base, w = 1 << 20, 1 << 24   # an activation range and a parameter range far away from it
    f = ctypes.c_float
    # [2, 64, 16] fp16 = 4096 bytes
    gn = lambda x, y: lib.msd_groupnorm(p(x), p(y), p(w), p(w), 2, 64, 16, 32, f(1e-5), 1, 1, None)
    assert gn(base, base + 2048) == 1 and gn(base + 4094, base) == 1
    assert lib.msd_chunk_add_groupnorm(p(base), p(w), p(base + 64), p(w), p(w), 2, 64, 16, 32, f(1e-5), 1, 1, None) == 1
    # the per-(sample, channel) addend ([2, 64] fp16 = 256 bytes) inside the output, in place and apart
    far_y = base + (1 << 16)
    chunk_gn = lambda chunk, y: lib.msd_chunk_add_groupnorm(p(base), p(chunk), p(y), p(w), p(w), 2, 64, 16, 32,
                                                            f(1e-5), 1, 1, None)
    assert chunk_gn(base + 1024, base) == 1 and chunk_gn(far_y + 4094, far_y) == 1 and chunk_gn(far_y - 2, far_y) == 1
    tok = lambda x, y: lib.msd_groupnorm_tokens(p(x), p(y), p(w), p(w), 2, 64, 16, 32, f(1e-6), 1, None)
    assert tok(base, base) == 1 and tok(base, base + 4094) == 1 and tok(base + 2, base) == 1
    # [8, 64] fp32 = 2048 bytes
    ln = lambda x, y: lib.msd_layernorm(p(x), p(y), p(w), p(w), 8, 64, f(1e-5), 0, None)
    assert ln(base, base + 4) == 1 and ln(base + 2044, base) == 1
    addln = lambda a, b, s_, y: lib.msd_add_layernorm(p(a), p(b), p(s_), p(y), p(w), p(w), 8, 64, f(1e-5), 0, None)
    far = base + (1 << 16)
    assert addln(base, far, base + 8, far + 4096) == 1        # the sum shifted against a
    assert addln(base, far, far + 8, far + 4096) == 1         # ... against b
    assert addln(base, far, far + 4096, far + 4096) == 1      # the sum and the result in one place
    assert addln(base, far, far + 4096, far + 4100) == 1
    assert lib.msd_elemwise_add(p(base), p(far), p(base + 4), 512, 0, None) == 1
    assert lib.msd_elemwise_add(p(base), p(far), p(far + 2044), 512, 0, None) == 1
    assert lib.msd_chunkwise_add(p(base), p(w), p(base + 4), 512, 64, 0, None) == 1
    assert lib.msd_chunkwise_add(p(base), p(base + 2048 + 16), p(base + 2048), 512, 64, 0, None) == 1  # chunk inside c
    for act in (lib.msd_silu, lib.msd_gelu, lib.msd_quick_gelu):
        assert act(p(base), p(base + 2), 512, 1, None) == 1
    perm = lambda a, b: lib.msd_permute_0_2_1(p(a), p(b), 2, 16, 16, 1, None)   # 1024 bytes
    assert perm(base, base) == 1 and perm(base, base + 1022) == 1 and perm(base + 512, base) == 1
    # Linear: x [2, 8], y [2, 4] fp32
    lin = lambda x, y: lib.msd_linear_rows(p(x), p(w), None, p(y), 2, 4, 8, 0, 0, 0, None)
    assert lin(base, base) == 1 and lin(base, base + 60) == 1 and lin(base + 28, base) == 1
    ys = (ctypes.c_void_p * 2)(far, base + 60)
    ws = (ctypes.c_void_p * 2)(w, w)
    ns = (ctypes.c_size_t * 2)(4, 4)
    assert lib.msd_linear_rows_grouped(p(base), ws, None, ys, ns, 2, 2, 8, 0, 0, 0, None) == 1
    # the problems of a grouped launch run side by side: outputs ([2, 4] fp32 = 32 bytes) may not
    # overlap each other, nor any problem's weights ([4, 8] fp32 = 128 bytes) or bias (16 bytes)
    def grouped(y0, y1, w0=w, w1=w + 4096, b0=None, b1=None):
        ys_ = (ctypes.c_void_p * 2)(y0, y1)
        ws_ = (ctypes.c_void_p * 2)(w0, w1)
        bs_ = None if b0 is None and b1 is None else (ctypes.c_void_p * 2)(b0, b1)
        return lib.msd_linear_rows_grouped(p(base), ws_, bs_, ys_, ns, 2, 2, 8, 0, 0, 0, None)
    assert grouped(far, far) == 1 and grouped(far, far + 28) == 1                 # output in output
    assert grouped(far, far + 64, w1=far - 64) == 1                               # output 0 in the weights of problem 1
    assert grouped(far, far + 64, w0=far + 32) == 1                               # output 1 in the weights of problem 0
    assert grouped(far, far + 64, b0=far + 4096, b1=far + 72) == 1                # output 1 in a bias
    assert lib.msd_linear_rows_grouped(p(base), ws, None, ys, ns, 2, 2, (1 << 28) + 8, 0, 0, 0, None) == 1  # k too long
    assert lib.msd_softmax(p(base), p(base + 2), 4, 77, 0, 1, None) == 1
    upd = lambda x, e, y: lib.msd_ddim_update(p(x), p(e), p(y), 64, f(0.5), f(0.6), f(0.7), 0, None)
    assert upd(base, far, base + 4) == 1 and upd(base, far, far + 252) == 1
    # sizes whose byte count does not fit are refused as well
    huge = (1 << 62)
    assert lib.msd_silu(p(base), p(far), huge, 0, None) == 1
    assert lib.msd_permute_0_2_1(p(base), p(far), 1 << 31, 1 << 31, 8, 1, None) == 1
    assert lib.msd_groupnorm(p(base), p(far), p(w), p(w), 1 << 40, 32, 1 << 30, 32, f(1e-5), 0, 0, None) == 1
    assert lib.msd_geglu(p(base), p(far), 1 << 40, 1 << 30, 1, None) == 1
    assert lib.msd_geglu(p(base), p(far), 1 << 31, 1 << 29, 0, None) == 1         # 2 * rows * inner * 4 bytes: 2^63


def test_stream_per_thread_is_refused_for_every_groupnorm_that_may_use_the_stream_scratch(msd):
    """hipStreamPerThread names a different stream in every thread, so it cannot key the
    per-stream scratch: the calls that may need that scratch refuse it whatever the shape (a
    small unit that would not be cut as well as a large one), before anything is launched."""
    lib = msd.load_library()
    p, f = ctypes.c_void_p, ctypes.c_float
    per_thread = p(2)  # the value of hipStreamPerThread
    x, y, w = 1 << 20, 1 << 22, 1 << 24
    for channels, hw in ((64, 16), (320, 4096)):
        assert lib.msd_groupnorm(p(x), p(y), p(w), p(w), 2, channels, hw, 32, f(1e-5), 1, 1, per_thread) == 1
        assert lib.msd_groupnorm(p(x), p(x), p(w), p(w), 2, channels, hw, 32, f(1e-5), 1, 1, per_thread) == 1
        assert lib.msd_chunk_add_groupnorm(p(x), p(w), p(y), p(w), p(w), 2, channels, hw, 32, f(1e-5), 1, 1,
                                           per_thread) == 1
        assert lib.msd_groupnorm_tokens(p(x), p(y), p(w), p(w), 2, channels, hw, 32, f(1e-6), 1, per_thread) == 1


def test_missing_library_fails_loudly(msd):
    with pytest.raises(msd.MsdError):
        msd.load_library(os.path.join(REPO, "does_not_exist.so"))
