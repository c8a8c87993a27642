"""ctypes/numpy access to the CPU oracle (liboracle.so, built by oracle/Makefile).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py.  Never by the product package.
"""
import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_DIR, "liboracle.so")
_lib = None

_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(dtype=np.float64, flags="C_CONTIGUOUS")
_u16p = np.ctypeslib.ndpointer(dtype=np.uint16, flags="C_CONTIGUOUS")
_i64p = np.ctypeslib.ndpointer(dtype=np.int64, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
_sz = ctypes.c_size_t
_fl = ctypes.c_float
_db = ctypes.c_double
_it = ctypes.c_int
_u64 = ctypes.c_uint64
_i64 = ctypes.c_int64


def build():
    subprocess.run(["make", "-C", _DIR, "-B"], check=True, stdout=subprocess.PIPE,
                   stderr=subprocess.STDOUT)
    return LIB_PATH


def build_flags():
    """The compiler flags of liboracle.so as oracle/Makefile states them."""
    try:
        for line in open(os.path.join(_DIR, "Makefile")):
            if line.startswith("CFLAGS"):
                return "gcc " + line.split(":=", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        build()
    L = ctypes.CDLL(LIB_PATH)
    sig = {
        "orc_fill_normal": (None, [_f32p, _sz, _u64, _fl, _fl]),
        "orc_add_outliers": (None, [_f32p, _sz, _u64, _fl]),
        "orc_fill_uniform_int": (None, [_i64p, _sz, _u64, _i64, _i64]),
        "orc_round_to_half": (None, [_f32p, _sz]),
        "orc_to_half_bits": (None, [_f32p, _u16p, _sz]),
        "orc_from_half_bits": (None, [_u16p, _f32p, _sz]),
        "orc_local_reduction_mean": (None, [_f32p, _f32p, _sz, _sz]),
        "orc_local_reduction_variance": (None, [_f32p, _f32p, _f32p, _sz, _sz]),
        "orc_group_norm": (None, [_f32p, _f32p, _f32p, _f32p, _f32p, _sz, _sz, _fl, _f32p, _sz]),
        "orc_layer_norm": (None, [_f32p, _f32p, _f32p, _f32p, _f32p, _sz, _fl, _f32p, _sz]),
        "orc_silu": (None, [_f32p, _f32p, _sz]),
        "orc_gelu": (None, [_f32p, _f32p, _sz]),
        "orc_quick_gelu": (None, [_f32p, _f32p, _sz]),
        "orc_gelu_multiply": (None, [_f32p, _f32p, _sz, _sz]),
        "orc_elemwise_add": (None, [_f32p, _f32p, _f32p, _sz]),
        "orc_chunkwise_add": (None, [_f32p, _f32p, _f32p, _sz, _sz]),
        "orc_permute3D_0_2_1": (None, [_f32p, _f32p, _sz, _sz, _sz]),
        "orc_timestep_embedding": (None, [_i64, _f32p, _it, _fl]),
        "orc_timestep_freqs": (None, [_f32p, _it, _fl]),
        "orc_ddim_timesteps": (_it, [_it, _i32p, _it]),
        "orc_groupnorm_forward": (_it, [_f32p, _f32p, _f32p, _f32p, _sz, _sz, _sz, _sz, _fl, _it]),
        "orc_layernorm_forward": (_it, [_f32p, _f32p, _f32p, _f32p, _sz, _sz, _fl]),
        "orc64_groupnorm": (None, [_f32p, _f64p, _f32p, _f32p, _sz, _sz, _sz, _sz, _db, _it]),
        "orc64_layernorm": (None, [_f32p, _f64p, _f32p, _f32p, _sz, _sz, _db]),
        "orc64_silu": (None, [_f32p, _f64p, _sz]),
        "orc64_gelu": (None, [_f32p, _f64p, _sz]),
        "orc64_quick_gelu": (None, [_f32p, _f64p, _sz]),
        "orc64_geglu": (None, [_f32p, _f64p, _sz, _sz]),
        "orc64_timestep_embedding": (None, [_i64, _f64p, _it, _db]),
        "orc_linear": (None, [_f32p, _f32p, ctypes.c_void_p, _f32p, _sz, _sz, _sz]),
        "orc64_linear": (None, [_f32p, _f32p, ctypes.c_void_p, _f64p, _sz, _sz, _sz]),
        "orc_softmax": (None, [_f32p, _f32p, _sz, _sz, _sz]),
        "orc64_softmax": (None, [_f32p, _f64p, _sz, _sz]),
        "orc_alphas_cumprod": (None, [_f32p]),
        "orc_ddim_schedule": (_it, [_it, _i32p, _f32p, _f32p, _f32p, _it]),
        "orc_ddim_update": (None, [_f32p, _f32p, _f32p, _sz, _fl, _fl, _fl]),
        "orc64_ddim_update": (None, [_f32p, _f32p, _f64p, _sz, _db, _db]),
        "orc_max_threads": (_it, []),
        "orc_set_threads": (None, [_it]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


# ---------------------------------------------------------------- data
def normal(shape, seed, mean=0.0, sigma=1.0):
    out = np.empty(shape, dtype=np.float32)
    lib().orc_fill_normal(out.reshape(-1), out.size, seed, mean, sigma)
    return out


def add_outliers(x, seed, magnitude=20.0):
    flat = x.reshape(-1)
    lib().orc_add_outliers(flat, flat.size, seed, magnitude)
    return x


def uniform_int(n, seed, lo, hi):
    out = np.empty(n, dtype=np.int64)
    lib().orc_fill_uniform_int(out, n, seed, lo, hi)
    return out


def round_to_half(x):
    y = np.ascontiguousarray(x, dtype=np.float32).copy()
    lib().orc_round_to_half(y.reshape(-1), y.size)
    return y


def to_half_bits(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    h = np.empty(x.shape, dtype=np.uint16)
    lib().orc_to_half_bits(x.reshape(-1), h.reshape(-1), x.size)
    return h


def from_half_bits(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    x = np.empty(h.shape, dtype=np.float32)
    lib().orc_from_half_bits(h.reshape(-1), x.reshape(-1), h.size)
    return x


# ---------------------------------------------------------------- float32 restatements
def groupnorm(x, weight, bias, groups, eps=1e-5, silu=False):
    """x: [batch, C, ...] float32.  Raises ValueError on a reference precondition."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    batch, channels = x.shape[0], x.shape[1]
    hw = x.size // (batch * channels)
    y = np.empty_like(x)
    rc = lib().orc_groupnorm_forward(x.reshape(-1), y.reshape(-1), _c(weight), _c(bias), batch,
                                     channels, hw, groups, eps, int(silu))
    if rc != 0:
        raise ValueError("reference GroupNorm precondition violated")
    return y


def layernorm(x, weight, bias, eps=1e-5):
    x = np.ascontiguousarray(x, dtype=np.float32)
    dim = x.shape[-1]
    y = np.empty_like(x)
    rc = lib().orc_layernorm_forward(x.reshape(-1), y.reshape(-1), _c(weight), _c(bias),
                                     x.size // dim, dim, eps)
    if rc != 0:
        raise ValueError("reference LayerNorm precondition violated")
    return y


def _c(a):
    return np.ascontiguousarray(a, dtype=np.float32).reshape(-1)


def _unary(name, x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty_like(x)
    getattr(lib(), name)(x.reshape(-1), y.reshape(-1), x.size)
    return y


def silu(x):
    return _unary("orc_silu", x)


def gelu(x):
    return _unary("orc_gelu", x)


def quick_gelu(x):
    return _unary("orc_quick_gelu", x)


def geglu(ab):
    ab = np.ascontiguousarray(ab, dtype=np.float32)
    inner = ab.shape[-1] // 2
    rows = ab.size // (2 * inner)
    y = np.empty(ab.shape[:-1] + (inner,), dtype=np.float32)
    lib().orc_gelu_multiply(ab.reshape(-1), y.reshape(-1), rows, inner)
    return y


def elemwise_add(a, b):
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    c = np.empty_like(a)
    lib().orc_elemwise_add(a.reshape(-1), b.reshape(-1), c.reshape(-1), a.size)
    return c


def chunkwise_add(a, chunk, chunk_size):
    """a: any shape; chunk: flat, one value per run of chunk_size elements of a."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    c = np.empty_like(a)
    lib().orc_chunkwise_add(a.reshape(-1), _c(chunk), c.reshape(-1), a.size, chunk_size)
    return c


def permute_0_2_1(x):
    """[i, j, k] -> [i, k, j]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    i, j, k = x.shape
    y = np.empty((i, k, j), dtype=np.float32)
    lib().orc_permute3D_0_2_1(x.reshape(-1), y.reshape(-1), i, j, k)
    return y


def timestep_embedding(t, dim=320, max_period=10000.0):
    out = np.empty(dim, dtype=np.float32)
    lib().orc_timestep_embedding(int(t), out, dim, max_period)
    return out


def timestep_freqs(half=160, max_period=10000.0):
    out = np.empty(half, dtype=np.float32)
    lib().orc_timestep_freqs(out, half, max_period)
    return out


def ddim_timesteps(steps):
    buf = np.zeros(1001, dtype=np.int32)
    n = lib().orc_ddim_timesteps(steps, buf, buf.size)
    if n < 0:
        raise ValueError("steps out of range")
    return buf[:n].tolist()


# ---------------------------------------------------------------- neighbours of the path
def _bias_ptr(bias):
    if bias is None:
        return None, None
    b = np.ascontiguousarray(bias, dtype=np.float32).reshape(-1)
    return b, b.ctypes.data_as(ctypes.c_void_p)


def linear(x, weight, bias=None):
    """x [m, k], weight [n, k] -> [m, n] (float32, k ascending)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(weight, dtype=np.float32)
    m, k = x.shape
    n = w.shape[0]
    assert w.shape[1] == k
    y = np.empty((m, n), dtype=np.float32)
    keep, bp = _bias_ptr(bias)
    lib().orc_linear(x.reshape(-1), w.reshape(-1), bp, y.reshape(-1), m, n, k)
    return y


def linear64(x, weight, bias=None):
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(weight, dtype=np.float32)
    m, k = x.shape
    n = w.shape[0]
    y = np.empty((m, n), dtype=np.float64)
    keep, bp = _bias_ptr(bias)
    lib().orc64_linear(x.reshape(-1), w.reshape(-1), bp, y.reshape(-1), m, n, k)
    return y


def softmax(x, local_size=64):
    """Row softmax over the last axis as the reference computes it (no max subtraction)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    chunk = x.shape[-1]
    y = np.empty_like(x)
    lib().orc_softmax(x.reshape(-1), y.reshape(-1), x.size // chunk, chunk, local_size)
    return y


def softmax64(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    chunk = x.shape[-1]
    y = np.empty(x.shape, dtype=np.float64)
    lib().orc64_softmax(x.reshape(-1), y.reshape(-1), x.size // chunk, chunk)
    return y


def alphas_cumprod():
    out = np.empty(1000, dtype=np.float32)
    lib().orc_alphas_cumprod(out)
    return out


def ddim_schedule(steps):
    """-> (timesteps, alphas, alphas_prev, sqrt_one_minus_alphas); ValueError as the C code says."""
    ts = np.zeros(1001, dtype=np.int32)
    a = np.zeros(1001, dtype=np.float32)
    ap = np.zeros(1001, dtype=np.float32)
    s1m = np.zeros(1001, dtype=np.float32)
    n = lib().orc_ddim_schedule(steps, ts, a, ap, s1m, 1001)
    if n < 0:
        raise ValueError("steps out of range" if n == -1 else "timestep list reaches 1000")
    return ts[:n].copy(), a[:n].copy(), ap[:n].copy(), s1m[:n].copy()


def ddim_update(x, e_t, a_t, a_prev, sqrt_one_minus_at):
    x = np.ascontiguousarray(x, dtype=np.float32)
    e = np.ascontiguousarray(e_t, dtype=np.float32)
    y = np.empty_like(x)
    lib().orc_ddim_update(x.reshape(-1), e.reshape(-1), y.reshape(-1), x.size, a_t, a_prev,
                          sqrt_one_minus_at)
    return y


def ddim_update64(x, e_t, a_t, a_prev):
    x = np.ascontiguousarray(x, dtype=np.float32)
    e = np.ascontiguousarray(e_t, dtype=np.float32)
    y = np.empty(x.shape, dtype=np.float64)
    lib().orc64_ddim_update(x.reshape(-1), e.reshape(-1), y.reshape(-1), x.size, a_t, a_prev)
    return y


# ---------------------------------------------------------------- float64 textbook
def groupnorm64(x, weight, bias, groups, eps=1e-5, silu=False):
    x = np.ascontiguousarray(x, dtype=np.float32)
    batch, channels = x.shape[0], x.shape[1]
    y = np.empty(x.shape, dtype=np.float64)
    lib().orc64_groupnorm(x.reshape(-1), y.reshape(-1), _c(weight), _c(bias), batch, channels,
                          x.size // (batch * channels), groups, eps, int(silu))
    return y


def layernorm64(x, weight, bias, eps=1e-5):
    x = np.ascontiguousarray(x, dtype=np.float32)
    dim = x.shape[-1]
    y = np.empty(x.shape, dtype=np.float64)
    lib().orc64_layernorm(x.reshape(-1), y.reshape(-1), _c(weight), _c(bias), x.size // dim, dim, eps)
    return y


def _unary64(name, x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty(x.shape, dtype=np.float64)
    getattr(lib(), name)(x.reshape(-1), y.reshape(-1), x.size)
    return y


def silu64(x):
    return _unary64("orc64_silu", x)


def gelu64(x):
    return _unary64("orc64_gelu", x)


def quick_gelu64(x):
    return _unary64("orc64_quick_gelu", x)


def geglu64(ab):
    ab = np.ascontiguousarray(ab, dtype=np.float32)
    inner = ab.shape[-1] // 2
    y = np.empty(ab.shape[:-1] + (inner,), dtype=np.float64)
    lib().orc64_geglu(ab.reshape(-1), y.reshape(-1), ab.size // (2 * inner), inner)
    return y


def timestep_embedding64(t, dim=320, max_period=10000.0):
    out = np.empty(dim, dtype=np.float64)
    lib().orc64_timestep_embedding(int(t), out, dim, max_period)
    return out


def max_threads():
    return lib().orc_max_threads()


def set_threads(n):
    lib().orc_set_threads(n)
