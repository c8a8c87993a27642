"""ctypes access to the MI355X norm / activation / embedding library.

The product is the native code under csrc/ (HIP kernels behind the C ABI of
include/msd_hip.h, and the C++ layer objects on top of it).  This module only
loads the built libraries and passes torch tensors' device pointers and the
current torch stream through the C ABI; torch is used for device memory and
streams, nothing else.  There is no fallback: if the library was not built
the loader raises.
"""
import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(_PKG_DIR, "csrc")
LIB_HIP_PATH = os.path.join(CSRC_DIR, "libmsd_hip.so")
LIB_NN_PATH = os.path.join(CSRC_DIR, "libmsd_nn.so")

DTYPE_F32 = 0
DTYPE_F16 = 1
TUNE_GN_SPLIT, TUNE_GN_THREADS, TUNE_LN_CHUNK, TUNE_LN_THREADS, TUNE_GEGLU_VECTORS, TUNE_ACT_VECTORS, \
    TUNE_SOFTMAX_ROWS, TUNE_GN_SPIN_LIMIT, TUNE_GN_WRITERS, TUNE_DEVICE_CUS, TUNE_DEVICE_XCDS, \
    TUNE_GN_PLAN_RULE_ONLY = range(12)
ERR_SCRATCH_LIMIT = -2

# every symbol include/msd_hip.h declares
C_ABI_SYMBOLS = (
    "msd_version", "msd_error_string", "msd_init", "msd_release", "msd_shutdown", "msd_status",
    "msd_gn_fallbacks", "msd_set_tuning", "msd_groupnorm", "msd_groupnorm_noalloc", "msd_groupnorm_plan", "msd_layernorm", "msd_geglu",
    "msd_silu", "msd_gelu", "msd_quick_gelu", "msd_timestep_embedding", "msd_ddim_timesteps",
    "msd_elemwise_add", "msd_chunkwise_add", "msd_chunk_add_groupnorm", "msd_add_layernorm", "msd_copy",
    "msd_groupnorm_tokens", "msd_permute_0_2_1",
    "msd_linear_rows", "msd_linear_rows_grouped", "msd_softmax", "msd_alphas_cumprod", "msd_ddim_schedule", "msd_ddim_update",
)
ACT_NONE, ACT_SILU = 0, 1

_lib = None


class MsdError(RuntimeError):
    pass


def load_library(path=None):
    """Loads libmsd_hip.so (built in-tree) and declares the C ABI signatures."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    path = path or LIB_HIP_PATH
    if not os.path.exists(path):
        raise MsdError(
            "native library %s is missing: build it with `python -c 'import __graft_entry__ as g;"
            " g.build()'` (there is no non-native fallback)" % path)
    lib = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
    vp, sz, fl, it = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float, ctypes.c_int
    lib.msd_version.restype = it
    lib.msd_error_string.restype = ctypes.c_char_p
    lib.msd_error_string.argtypes = [it]
    lib.msd_init.argtypes = [vp]
    lib.msd_shutdown.argtypes = []
    lib.msd_status.argtypes = [vp]
    lib.msd_release.argtypes = [vp]
    lib.msd_gn_fallbacks.argtypes = [vp, ctypes.POINTER(ctypes.c_uint), it]
    lib.msd_set_tuning.argtypes = [it, it]
    lib.msd_groupnorm.argtypes = [vp, vp, vp, vp, sz, sz, sz, sz, fl, it, it, vp]
    lib.msd_groupnorm_noalloc.argtypes = [vp, vp, vp, vp, sz, sz, sz, sz, fl, it, it, vp]
    lib.msd_groupnorm_plan.argtypes = [sz, sz, sz, sz, it, it, it] + [ctypes.POINTER(ctypes.c_int)] * 4
    lib.msd_layernorm.argtypes = [vp, vp, vp, vp, sz, sz, fl, it, vp]
    lib.msd_geglu.argtypes = [vp, vp, sz, sz, it, vp]
    lib.msd_copy.argtypes = [vp, vp, sz, vp]
    lib.msd_permute_0_2_1.argtypes = [vp, vp, sz, sz, sz, it, vp]
    lib.msd_groupnorm_tokens.argtypes = [vp, vp, vp, vp, sz, sz, sz, sz, fl, it, vp]
    lib.msd_elemwise_add.argtypes = [vp, vp, vp, sz, it, vp]
    lib.msd_chunkwise_add.argtypes = [vp, vp, vp, sz, sz, it, vp]
    lib.msd_chunk_add_groupnorm.argtypes = [vp, vp, vp, vp, vp, sz, sz, sz, sz, fl, it, it, vp]
    lib.msd_add_layernorm.argtypes = [vp, vp, vp, vp, vp, vp, sz, sz, fl, it, vp]
    for name in ("msd_silu", "msd_gelu", "msd_quick_gelu"):
        getattr(lib, name).argtypes = [vp, vp, sz, it, vp]
    lib.msd_timestep_embedding.argtypes = [vp, vp, sz, sz, fl, it, vp]
    lib.msd_ddim_timesteps.argtypes = [it, ctypes.POINTER(ctypes.c_int), it]
    lib.msd_linear_rows.argtypes = [vp, vp, vp, vp, sz, sz, sz, it, it, it, vp]
    lib.msd_softmax.argtypes = [vp, vp, sz, sz, it, it, vp]
    lib.msd_linear_rows_grouped.argtypes = [vp, ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.POINTER(vp),
                                            ctypes.POINTER(sz), sz, sz, sz, it, it, it, vp]
    flp, inp = ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_int)
    lib.msd_alphas_cumprod.argtypes = [flp]
    lib.msd_ddim_schedule.argtypes = [it, inp, flp, flp, flp, it]
    lib.msd_ddim_update.argtypes = [vp, vp, vp, sz, fl, fl, fl, it, vp]
    for name in C_ABI_SYMBOLS:
        if name != "msd_error_string":
            getattr(lib, name).restype = it
    _lib = lib
    return lib


def check(code):
    if code != 0:
        raise MsdError("msd call failed with code %d: %s"
                       % (code, load_library().msd_error_string(code).decode()))


def _dtype_code(t):
    import torch
    if t.dtype == torch.float32:
        return DTYPE_F32
    if t.dtype == torch.float16:
        return DTYPE_F16
    raise MsdError("unsupported storage dtype %s" % t.dtype)


def _stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev(t):
    if not t.is_cuda or not t.is_contiguous():
        raise MsdError("expected a contiguous device tensor")
    return ctypes.c_void_p(t.data_ptr())


def _affine(t, n, like, what):
    """gamma / beta / bias: float32, n values, on the device of `like`."""
    import torch
    if t.dtype != torch.float32 or t.numel() != n or t.device != like.device:
        raise MsdError("%s must be float32 with %d values on %s (got %s, %d, %s)"
                       % (what, n, like.device, t.dtype, t.numel(), t.device))
    return _dev(t)


def _same(t, like, numel, what):
    """An output / second operand: dtype and device of `like`, `numel` elements."""
    if t.dtype != like.dtype or t.device != like.device or t.numel() != numel:
        raise MsdError("%s must be %s with %d elements on %s (got %s, %d, %s)"
                       % (what, like.dtype, numel, like.device, t.dtype, t.numel(), t.device))
    return _dev(t)


def init():
    check(load_library().msd_init(_stream()))


def status():
    return load_library().msd_status(_stream())


def gn_fallbacks(reset=False):
    """How often a GroupNorm workgroup computed a sibling's statistics itself (diagnostic)."""
    n = ctypes.c_uint(0)
    check(load_library().msd_gn_fallbacks(_stream(), ctypes.byref(n), int(reset)))
    return n.value


def groupnorm(x, gamma, beta, groups, eps=1e-5, fuse_silu=False, out=None, noalloc=False):
    """x: [batch, C, ...] device tensor; gamma/beta float32 [C]; out may be x (in place).
    noalloc: go through msd_groupnorm_noalloc (fixed scratch, batch * groups <= 1024)."""
    import torch
    out = torch.empty_like(x) if out is None else out
    batch, channels = x.shape[0], x.shape[1]
    hw = x.numel() // (batch * channels) if batch * channels else 0
    fn = load_library().msd_groupnorm_noalloc if noalloc else load_library().msd_groupnorm
    check(fn(_dev(x), _same(out, x, x.numel(), "out"), _affine(gamma, channels, x, "gamma"),
             _affine(beta, channels, x, "beta"), batch, channels, hw, groups, eps, int(fuse_silu),
             _dtype_code(x), _stream()))
    return out


def groupnorm_plan(batch, channels, hw, groups=32, dtype_code=DTYPE_F16, noalloc=False, in_place=False):
    """(split, threads, vectors per lane, writers) of the launch msd_groupnorm makes for this
    shape; (0, 0, 0, 1) = the general kernel; writers > 1 = that many workgroups share each whole
    (sample, group) and store a part of it each (never for a call in place).  Host arithmetic,
    no GPU needed."""
    out = [ctypes.c_int(0) for _ in range(4)]
    check(load_library().msd_groupnorm_plan(batch, channels, hw, groups, dtype_code, int(noalloc), int(in_place),
                                            *[ctypes.byref(o) for o in out]))
    return tuple(o.value for o in out)


def groupnorm_tokens(x, gamma, beta, groups, eps=1e-6):
    """x: [batch, C, ...] -> [batch, H*W, C] = GroupNorm(x) with channels last (no SiLU)."""
    import torch
    batch, channels = x.shape[0], x.shape[1]
    hw = x.numel() // (batch * channels) if batch * channels else 0
    out = torch.empty((batch, hw, channels), dtype=x.dtype, device=x.device)
    check(load_library().msd_groupnorm_tokens(_dev(x), _dev(out), _affine(gamma, channels, x, "gamma"),
                                              _affine(beta, channels, x, "beta"), batch, channels,
                                              hw, groups, eps, _dtype_code(x), _stream()))
    return out


def permute_0_2_1(x):
    """[i, j, k] -> [i, k, j] (new tensor)."""
    import torch
    i, j, k = x.shape
    out = torch.empty((i, k, j), dtype=x.dtype, device=x.device)
    check(load_library().msd_permute_0_2_1(_dev(x), _dev(out), i, j, k, _dtype_code(x), _stream()))
    return out


def chunk_add_groupnorm(x, chunk, gamma, beta, groups, eps=1e-5, fuse_silu=False, out=None):
    """GroupNorm(x + chunk[:, :, None]) (+ SiLU); chunk: [batch, C] in x's dtype."""
    import torch
    out = torch.empty_like(x) if out is None else out
    batch, channels = x.shape[0], x.shape[1]
    hw = x.numel() // (batch * channels) if batch * channels else 0
    check(load_library().msd_chunk_add_groupnorm(_dev(x), _same(chunk, x, batch * channels, "chunk"),
                                                 _same(out, x, x.numel(), "out"),
                                                 _affine(gamma, channels, x, "gamma"), _affine(beta, channels, x, "beta"),
                                                 batch, channels, hw, groups, eps, int(fuse_silu),
                                                 _dtype_code(x), _stream()))
    return out


def add_layernorm(a, b, gamma, beta, eps=1e-5, sum_out=None, out=None):
    """Returns (a + b, LayerNorm(a + b)); sum_out may be a or b."""
    import torch
    sum_out = torch.empty_like(a) if sum_out is None else sum_out
    out = torch.empty_like(a) if out is None else out
    dim = a.shape[-1]
    rows = a.numel() // dim if dim else 0
    check(load_library().msd_add_layernorm(_dev(a), _same(b, a, a.numel(), "b"), _same(sum_out, a, a.numel(), "sum_out"),
                                           _same(out, a, a.numel(), "out"), _affine(gamma, dim, a, "gamma"),
                                           _affine(beta, dim, a, "beta"), rows, dim, eps, _dtype_code(a), _stream()))
    return sum_out, out


def elemwise_add(a, b, out=None):
    import torch
    out = torch.empty_like(a) if out is None else out
    check(load_library().msd_elemwise_add(_dev(a), _same(b, a, a.numel(), "b"), _same(out, a, a.numel(), "out"),
                                          a.numel(), _dtype_code(a), _stream()))
    return out


def chunkwise_add(a, chunk, chunk_size, out=None):
    import torch
    out = torch.empty_like(a) if out is None else out
    if chunk_size <= 0 or a.numel() % chunk_size:
        raise MsdError("chunk_size must divide the element count")
    check(load_library().msd_chunkwise_add(_dev(a), _same(chunk, a, a.numel() // chunk_size, "chunk"),
                                           _same(out, a, a.numel(), "out"), a.numel(), chunk_size,
                                           _dtype_code(a), _stream()))
    return out


def layernorm(x, gamma, beta, eps=1e-5, out=None):
    import torch
    out = torch.empty_like(x) if out is None else out
    dim = x.shape[-1]
    rows = x.numel() // dim if dim else 0
    check(load_library().msd_layernorm(_dev(x), _same(out, x, x.numel(), "out"), _affine(gamma, dim, x, "gamma"),
                                       _affine(beta, dim, x, "beta"), rows, dim, eps,
                                       _dtype_code(x), _stream()))
    return out


def geglu(proj, out=None):
    """proj: [..., 2*inner] (value | gate) -> [..., inner]."""
    import torch
    inner = proj.shape[-1] // 2
    rows = proj.numel() // (2 * inner) if inner else 0
    if out is None:
        out = torch.empty(proj.shape[:-1] + (inner,), dtype=proj.dtype, device=proj.device)
    check(load_library().msd_geglu(_dev(proj), _same(out, proj, rows * inner, "out"), rows, inner,
                                   _dtype_code(proj), _stream()))
    return out


def _act(name, x, out):
    import torch
    out = torch.empty_like(x) if out is None else out
    check(getattr(load_library(), name)(_dev(x), _same(out, x, x.numel(), "out"), x.numel(), _dtype_code(x),
                                        _stream()))
    return out


def silu(x, out=None):
    return _act("msd_silu", x, out)


def gelu(x, out=None):
    return _act("msd_gelu", x, out)


def quick_gelu(x, out=None):
    return _act("msd_quick_gelu", x, out)


def timestep_embedding(timesteps, dim, max_period=10000.0, dtype=None):
    """timesteps: int64 device tensor [batch] -> [batch, dim] as [cos | sin]."""
    import torch
    dtype = dtype or torch.float32
    out = torch.empty((timesteps.numel(), dim), dtype=dtype, device=timesteps.device)
    check(load_library().msd_timestep_embedding(_dev(timesteps), _dev(out), timesteps.numel(), dim,
                                                max_period, _dtype_code(out), _stream()))
    return out


def ddim_timesteps(steps):
    """Ascending integer DDIM timestep list (host only)."""
    lib = load_library()
    n = lib.msd_ddim_timesteps(steps, None, 0)
    if n < 0:
        raise MsdError("ddim steps must be in [1, 1000]")
    buf = (ctypes.c_int * n)()
    lib.msd_ddim_timesteps(steps, buf, n)
    return list(buf)


def linear_rows(x, weight, bias=None, act_in=ACT_NONE, act_out=ACT_NONE, out=None):
    """x [m <= 8, k], weight [n, k] (x's dtype), bias float32 [n] or None -> [m, n]."""
    import torch
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k or weight.dtype != x.dtype:
        raise MsdError("weight must be [n, k] in the dtype of x")
    out = torch.empty((m, n), dtype=x.dtype, device=x.device) if out is None else out
    if weight.device != x.device:
        raise MsdError("weight and x must share a device")
    bp = _affine(bias, n, x, "bias") if bias is not None else None
    check(load_library().msd_linear_rows(_dev(x), _dev(weight), bp, _same(out, x, m * n, "out"), m, n, k, act_in, act_out,
                                         _dtype_code(x), _stream()))
    return out


def linear_rows_grouped(x, weights, biases=None, act_in=ACT_NONE, act_out=ACT_NONE):
    """One launch for several Linear layers on the same x [m <= 8, k]: weights[i] is [n_i, k] in
    x's dtype, biases[i] float32 [n_i] or None -> list of [m, n_i] tensors."""
    import torch
    m, k = x.shape
    count = len(weights)
    outs, wp, bp, yp, ns = [], (ctypes.c_void_p * count)(), (ctypes.c_void_p * count)(), \
        (ctypes.c_void_p * count)(), (ctypes.c_size_t * count)()
    for i, w in enumerate(weights):
        if w.dim() != 2 or w.shape[1] != k or w.dtype != x.dtype or w.device != x.device:
            raise MsdError("weights[%d] must be [n, %d] in the dtype and on the device of x" % (i, k))
        n = w.shape[0]
        out = torch.empty((m, n), dtype=x.dtype, device=x.device)
        outs.append(out)
        wp[i], yp[i], ns[i] = w.data_ptr() if w.numel() else None, out.data_ptr() if out.numel() else None, n
        b = biases[i] if biases is not None else None
        bp[i] = _affine(b, n, x, "biases[%d]" % i).value if b is not None else None
        if not w.is_contiguous():
            raise MsdError("expected contiguous weights")
    check(load_library().msd_linear_rows_grouped(_dev(x), wp, bp, yp, ns, count, m, k, act_in, act_out,
                                                 _dtype_code(x), _stream()))
    return outs


def softmax(x, stable=False, out=None):
    """Softmax over the last axis; out may be x (in place)."""
    import torch
    out = torch.empty_like(x) if out is None else out
    cols = x.shape[-1]
    rows = x.numel() // cols if cols else 0
    check(load_library().msd_softmax(_dev(x), _same(out, x, x.numel(), "out"), rows, cols, int(stable),
                                     _dtype_code(x), _stream()))
    return out


def alphas_cumprod():
    """The sampler's 1000 cumulative alpha products as a list of floats (host only)."""
    buf = (ctypes.c_float * 1000)()
    check(load_library().msd_alphas_cumprod(buf))
    return list(buf)


def ddim_schedule(steps):
    """-> (timesteps, alphas, alphas_prev, sqrt_one_minus_alphas) as lists (host only)."""
    lib = load_library()
    n = lib.msd_ddim_schedule(steps, None, None, None, None, 0)
    if n < 0:
        raise MsdError("ddim steps must be in [1, 500] (code %d)" % n)
    ts = (ctypes.c_int * n)()
    a, ap, s1m = (ctypes.c_float * n)(), (ctypes.c_float * n)(), (ctypes.c_float * n)()
    lib.msd_ddim_schedule(steps, ts, a, ap, s1m, n)
    return list(ts), list(a), list(ap), list(s1m)


def ddim_update(x, e_t, a_t, a_prev, sqrt_one_minus_at, out=None):
    """One DDIM step (eta 0) on device tensors; out may be x."""
    import torch
    out = torch.empty_like(x) if out is None else out
    check(load_library().msd_ddim_update(_dev(x), _same(e_t, x, x.numel(), "e_t"), _same(out, x, x.numel(), "out"),
                                         x.numel(), a_t, a_prev,
                                         sqrt_one_minus_at, _dtype_code(x), _stream()))
    return out


# ---------------------------------------------------------------------------------------
# C++ layer objects (libmsd_nn.so) through their plain-C handles
# ---------------------------------------------------------------------------------------
_nn = None
# int model(void *x, int t, void *e_t, size_t bytes, void *user): the sampler's noise-model callback
MODEL_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t,
                            ctypes.c_void_p)


def load_nn_library(path=None):
    """Loads libmsd_nn.so (GroupNorm / LayerNorm / GEGLU objects, NPY loader, step runner)."""
    global _nn
    if _nn is not None and path is None:
        return _nn
    load_library()
    path = path or LIB_NN_PATH
    if not os.path.exists(path):
        raise MsdError("native library %s is missing: run __graft_entry__.build()" % path)
    nn = ctypes.CDLL(path)
    vp, sz, fl, it, cp = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float, ctypes.c_int, ctypes.c_char_p
    szp = ctypes.POINTER(ctypes.c_size_t)
    flp = ctypes.POINTER(ctypes.c_float)
    lgp = ctypes.POINTER(ctypes.c_long)
    sig = {
        "msdnn_last_error": (cp, []),
        "msdnn_set_media_path": (None, [cp]),
        "msdnn_set_debug_timing": (None, [it]),
        "msdnn_npy_load": (it, [cp, flp, sz, szp, szp]),
        "msdnn_npy_save": (it, [cp, flp, sz]),
        "msdnn_groupnorm_create": (vp, [vp, sz, sz, fl, cp, cp, sz, it]),
        "msdnn_groupnorm_init": (it, [vp]),
        "msdnn_groupnorm_check": (it, [vp, sz, it]),
        "msdnn_groupnorm_forward": (it, [vp, vp, vp, sz, it]),
        "msdnn_groupnorm_forward_chunk": (it, [vp, vp, vp, sz, vp, sz, it]),
        "msdnn_groupnorm_forward_tokens": (it, [vp, vp, vp, sz, it]),
        "msdnn_groupnorm_destroy": (None, [vp]),
        "msdnn_layernorm_create": (vp, [vp, sz, cp, cp, fl]),
        "msdnn_layernorm_init": (it, [vp]),
        "msdnn_layernorm_check": (it, [vp, sz, it]),
        "msdnn_layernorm_forward": (it, [vp, vp, vp, sz, it]),
        "msdnn_layernorm_forward_add": (it, [vp, vp, vp, vp, vp, sz, it]),
        "msdnn_layernorm_destroy": (None, [vp]),
        "msdnn_geglu_create": (vp, [vp, sz, sz]),
        "msdnn_geglu_weight_shape": (it, [vp, szp, szp]),
        "msdnn_geglu_check": (it, [vp, sz, sz, it]),
        "msdnn_geglu_forward": (it, [vp, vp, sz, vp, sz, it]),
        "msdnn_geglu_destroy": (None, [vp]),
        "msdnn_activation": (it, [vp, it, vp, vp, sz, it]),
        "msdnn_timestep_embedding": (it, [vp, lgp, sz, flp]),
        "msdnn_ddim_timesteps": (it, [it, ctypes.POINTER(ctypes.c_int), it]),
        "msdnn_linear_create": (vp, [vp, sz, sz, cp, cp, it]),
        "msdnn_linear_init": (it, [vp]),
        "msdnn_linear_init_from": (it, [vp, flp, sz, flp, sz]),
        "msdnn_linear_forward": (it, [vp, vp, sz, vp, sz, it, it, it]),
        "msdnn_linear_forward_grouped": (it, [ctypes.POINTER(vp), sz, vp, sz, ctypes.POINTER(vp), szp, it, it, it]),
        "msdnn_linear_destroy": (None, [vp]),
        "msdnn_softmax": (it, [vp, vp, vp, sz, it, sz, it]),
        "msdnn_ddim_sample": (it, [vp, vp, sz, it, it, MODEL_FN, vp, vp]),
        "msdnn_ddim_make_schedule": (it, [ctypes.POINTER(ctypes.c_int), it, flp, flp]),
        "msdnn_test_buffer": (it, [vp, vp, sz, it, cp, flp, szp]),
        "msdnn_step_create": (vp, [vp, sz, it, it]),
        "msdnn_step_num_ops": (sz, [vp]),
        "msdnn_step_op_info": (it, [vp, sz, ctypes.POINTER(ctypes.c_int), szp, ctypes.POINTER(ctypes.c_int)]),
        "msdnn_step_download": (it, [vp, sz, it, flp, sz, szp]),
        "msdnn_step_affine": (it, [vp, sz, flp, flp, sz]),
        "msdnn_step_restore": (it, [vp]),
        "msdnn_step_bytes": (sz, [vp]),
        "msdnn_step_launches": (sz, [vp]),
        "msdnn_step_run": (it, [vp, it, it, lgp, sz]),
        "msdnn_step_destroy": (None, [vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(nn, name)
        fn.restype = res
        fn.argtypes = args
    _nn = nn
    return nn


def nn_last_error():
    return load_nn_library().msdnn_last_error().decode()
