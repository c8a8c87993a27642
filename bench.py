#!/usr/bin/env python3
"""Benchmark of the norm / activation / embedding path on one MI355X.

A "step" is one UNet step's worth of the hot path at batch 2 (CFG), fp16 storage:
the timestep embedding, 23 SiLU(emb), 45 GroupNorm(32)+SiLU (in- and out-norm of the
22 ResBlocks plus the final norm), 48 LayerNorms and 16 GEGLUs at their real shapes,
each layer on its own HBM-resident buffers, launched back to back on one stream.
`value` = algorithmic bytes of one step / time per step.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--mode graph|eager] [--no-cpu] [--no-shapes]
                    [--tables shapes,gn_split,fusions,neighbours,large_batch,gn_plan_sweep]
    python bench.py --sweep-summary OUT.json[,...]               (no GPU: markdown of gn_plan_sweep rows)
    python bench.py --trace-summary TRACE.csv --bench-json OUT [--plain-json OUT2]   (no GPU: shapes rows next to a kernel trace)

Prints ONE JSON line (see the keys below).  The CPU oracle is used only for the
`cpu_baseline` leg.
"""
import argparse
import importlib
import json
import os
import sys
import time

REPO = os.path.dirname(os.path.abspath(__file__))
if REPO not in sys.path:
    sys.path.insert(0, REPO)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
# HBM bytes per launch of each kernel family as the rocprofv3 FETCH_SIZE / WRITE_SIZE counters
# measured them (written next to the counter summary it was computed from)
TRAFFIC_JSON = os.path.join(REPO, "profiles", "traffic.json")


def measured_traffic():
    """{family: HBM bytes per launch} from profiles/traffic.json; {} when the file is absent."""
    try:
        with open(TRAFFIC_JSON) as f:
            return {k: v.get("traffic_bytes_per_launch") for k, v in json.load(f)["families"].items()}
    except (OSError, ValueError, KeyError):
        return {}


# ----------------------------------------------------------------------------
# The per-step workload (call order of UNetModel::forward, M/UNetModel.cpp:1078-1929)
# ----------------------------------------------------------------------------
# ResBlocks: (in_channels, out_channels, side) in execution order
RESBLOCKS = (
    [(320, 320, 64)] * 2 + [(320, 640, 32), (640, 640, 32), (640, 1280, 16), (1280, 1280, 16)] +
    [(1280, 1280, 8)] * 2 +                       # input blocks 10, 11
    [(1280, 1280, 8)] * 2 +                       # middle block
    [(2560, 1280, 8)] * 3 + [(2560, 1280, 16)] * 2 + [(1920, 1280, 16)] +
    [(1920, 640, 32), (1280, 640, 32), (960, 640, 32)] +
    [(960, 320, 64), (640, 320, 64), (640, 320, 64)]
)
# transformer blocks: (dim, tokens); 3 LayerNorms and 1 GEGLU each
TRANSFORMERS = [(320, 4096)] * 2 + [(640, 1024)] * 2 + [(1280, 256)] * 2 + [(1280, 64)] + \
               [(1280, 256)] * 3 + [(640, 1024)] * 3 + [(320, 4096)] * 3
BATCH = 2
ELT = 2  # fp16 storage


def step_layers():
    """List of (kind, params) in execution order for one UNet step."""
    layers = [("temb", {"dim": 320}), ("silu", {"n": BATCH * 1280})]  # time_embed MLP's SiLU
    tr = iter(TRANSFORMERS)
    # which ResBlocks are followed by a SpatialTransformer (M/UNetModel.cpp:86-1018)
    followed = [True, True, True, True, True, True, False, False,  # input blocks 1,2,4,5,7,8,10,11
                True, False,                                         # middle: res, ST, res
                False, False, False, True, True, True,               # output 0..5
                True, True, True, True, True, True]                  # output 6..11
    assert len(followed) == len(RESBLOCKS) == 22 and sum(followed) == 16
    for (cin, cout, side), st in zip(RESBLOCKS, followed):
        layers.append(("gn_silu", {"c": cin, "hw": side * side, "inplace": False}))
        layers.append(("silu", {"n": BATCH * 1280}))  # SiLU(emb) before the ResBlock's Linear
        layers.append(("gn_silu", {"c": cout, "hw": side * side, "inplace": True}))
        if st:
            dim, tokens = next(tr)
            assert tokens == side * side
            for _ in range(3):
                layers.append(("ln", {"rows": BATCH * tokens, "dim": dim}))
            layers.append(("geglu", {"rows": BATCH * tokens, "inner": 4 * dim}))
    layers.append(("gn_silu", {"c": 320, "hw": 4096, "inplace": True}))  # final norm + SiLU
    return layers


def layer_bytes(kind, p):
    """Algorithmic HBM bytes of one launch (gamma/beta excluded, as in the baseline table)."""
    if kind == "gn_silu":
        return 2 * BATCH * p["c"] * p["hw"] * ELT
    if kind == "ln":
        return 2 * p["rows"] * p["dim"] * ELT
    if kind == "geglu":
        return 3 * p["rows"] * p["inner"] * ELT
    return 0  # temb / SiLU(emb): a few KB, launch-bound, not counted


class Step:
    """Device buffers and launch closures for one step."""

    def __init__(self, msd, torch, dev, seed=5001, norms_in_place=True):
        self.msd, self.torch = msd, torch
        g = torch.Generator(device=dev).manual_seed(seed)
        self.launches = []
        self.bytes = 0
        self.by_kind = {}
        lib = msd.load_library()
        import ctypes
        vp = ctypes.c_void_p
        self._keep = []

        def randn(*shape, dtype=torch.float16):
            t = torch.randn(*shape, device=dev, dtype=torch.float32, generator=g).to(dtype)
            self._keep.append(t)
            return t

        # integer timesteps, uniform in [0, 999]
        self.t = torch.randint(0, 1000, (BATCH,), device=dev, dtype=torch.int64, generator=g)
        self._keep.append(self.t)
        affine = {}

        def gb(c):
            if c not in affine:
                affine[c] = (1.0 + 0.1 * randn(c, dtype=torch.float32), 0.1 * randn(c, dtype=torch.float32))
                self._keep.extend(affine[c])
            return affine[c]

        for kind, p in step_layers():
            nb = layer_bytes(kind, p)
            self.bytes += nb
            k = self.by_kind.setdefault(kind, {"launches": 0, "bytes": 0})
            k["launches"] += 1
            k["bytes"] += nb
            if kind == "temb":
                out = torch.empty((BATCH, p["dim"]), device=dev, dtype=torch.float16)
                self._keep.append(out)
                args = (vp(self.t.data_ptr()), vp(out.data_ptr()), BATCH, p["dim"], 10000.0, msd.DTYPE_F16)
                fn = lib.msd_timestep_embedding
            elif kind == "silu":
                x = randn(p["n"])
                args = (vp(x.data_ptr()), vp(x.data_ptr()), p["n"], msd.DTYPE_F16)
                fn = lib.msd_silu
            elif kind == "gn_silu":
                x = randn(BATCH, p["c"], p["hw"]) * 2.0
                self._keep.append(x)
                y = x if (p["inplace"] and norms_in_place) else torch.empty_like(x)
                self._keep.append(y)
                ga, be = gb(p["c"])
                args = (vp(x.data_ptr()), vp(y.data_ptr()), vp(ga.data_ptr()), vp(be.data_ptr()), BATCH,
                        p["c"], p["hw"], 32, 1e-5, 1, msd.DTYPE_F16)
                fn = lib.msd_groupnorm
            elif kind == "ln":
                x = randn(p["rows"], p["dim"])
                y = torch.empty_like(x)
                self._keep.append(y)
                ga, be = gb(p["dim"])
                args = (vp(x.data_ptr()), vp(y.data_ptr()), vp(ga.data_ptr()), vp(be.data_ptr()), p["rows"],
                        p["dim"], 1e-5, msd.DTYPE_F16)
                fn = lib.msd_layernorm
            elif kind == "geglu":
                x = randn(p["rows"], 2 * p["inner"])
                y = torch.empty((p["rows"], p["inner"]), device=dev, dtype=torch.float16)
                self._keep.append(y)
                args = (vp(x.data_ptr()), vp(y.data_ptr()), p["rows"], p["inner"], msd.DTYPE_F16)
                fn = lib.msd_geglu
            else:
                raise AssertionError(kind)
            self.launches.append((kind, fn, args))

    def run(self, stream_ptr, only=None):
        for kind, fn, args in self.launches:
            if only is None or kind == only:
                rc = fn(*args, stream_ptr)
                if rc != 0:
                    raise RuntimeError("%s failed: %d" % (kind, rc))


class CopyStep:
    """The same 133 launches with every kernel replaced by a plain 16-byte copy that moves the
    same number of bytes (read + write) between buffers of its own: what the launch structure
    and the tensor sizes alone cost on this machine."""

    def __init__(self, msd, torch, dev):
        import ctypes
        self.lib = msd.load_library()
        self.calls = []
        self._keep = []
        for kind, p in step_layers():
            nb = layer_bytes(kind, p)
            half = max(16, (nb // 2 + 15) // 16 * 16) if nb else 2 * BATCH * 1280  # bytes read = bytes written
            src = torch.empty(half, dtype=torch.uint8, device=dev)
            dst = torch.empty(half, dtype=torch.uint8, device=dev)
            src.random_(0, 255)
            self._keep += [src, dst]
            self.calls.append((ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst.data_ptr()), half))

    def run(self, stream_ptr):
        for src, dst, nbytes in self.calls:
            rc = self.lib.msd_copy(src, dst, nbytes, stream_ptr)
            if rc != 0:
                raise RuntimeError("copy failed: %d" % rc)


def timed_replays(torch, fn, reps):
    """Wall time (s) of `reps` calls of fn, bracketed by device synchronisation."""
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    return time.perf_counter() - t0


def event_time_ms(torch, fn, reps, batches=5):
    """Elapsed GPU time (ms) of `reps` calls of fn between two HIP events recorded on the
    stream the kernels are launched on (torch's current stream): the median of `batches`
    such measurements, each of reps / batches calls scaled back to `reps`."""
    per = max(1, reps // batches)
    times = []
    for _ in range(batches):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for _ in range(per):
            fn()
        b.record()
        b.synchronize()
        times.append(a.elapsed_time(b) / per)
    times.sort()
    return times[len(times) // 2] * reps


def capture(torch, msd, stream, body):
    """Captures body() (launches on the current stream) into a HIP graph; returns replay()."""
    import ctypes
    with torch.cuda.stream(stream):
        msd.check(msd.load_library().msd_init(ctypes.c_void_p(stream.cuda_stream)))  # scratch before capture
        body()  # warm: module load, scratch
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        body()
    torch.cuda.synchronize()
    return graph.replay


def _rotating_launch_us(torch, msd, stream, launch, xs, ys, warm=20, budget=2000):
    """µs per launch of `launch(x, y, stream_ptr)` over rotating buffer pairs, graph-replayed."""
    import ctypes
    copies = len(xs)

    def body():
        sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        for x, y in zip(xs, ys):
            assert launch(x, y, sp) == 0
    replay = capture(torch, msd, stream, body)
    reps = max(2, int(budget // copies))
    with torch.cuda.stream(stream):
        # at least `warm` warm-up launches and 20 ms of GPU work: the clocks have dropped while
        # the host was making this case's buffers
        t0 = time.perf_counter()
        done = 0
        while done < warm or time.perf_counter() - t0 < 0.02:
            for _ in range(warm // copies + 1):
                replay()
            done += (warm // copies + 1) * copies
            torch.cuda.synchronize()
        return event_time_ms(torch, replay, reps) * 1e3 / (reps * copies)


_HIP_RUNTIME = None


def hip_runtime():
    """ctypes handle of the HIP runtime this process already uses (the copy torch loaded, found
    in /proc/self/maps so that no second runtime is mapped), with hipMemcpyDtoDAsync declared."""
    global _HIP_RUNTIME
    if _HIP_RUNTIME is None:
        import ctypes
        path = None
        with open("/proc/self/maps") as f:
            for line in f:
                name = line.split()[-1]
                if "/libamdhip64.so" in name:
                    path = name
                    break
        if path is None:
            raise RuntimeError("the HIP runtime is not mapped into this process")
        rt = ctypes.CDLL(path)
        rt.hipMemcpyDtoDAsync.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        rt.hipMemcpyDtoDAsync.restype = ctypes.c_int
        _HIP_RUNTIME = rt
    return _HIP_RUNTIME


class TraceMarkers:
    """Numbers the timed measurements of a table so that a kernel trace of the same run can be cut
    into them: before measurement i one tiny launch of a kernel no table uses (quick_GELU on fp16)
    with i + 1 workgroups goes onto the stream; `labels[i]` says what was measured after it."""

    def __init__(self, torch, msd, dev):
        import ctypes
        self.labels = []
        self._lib = msd.load_library()
        self._code = msd.DTYPE_F16
        self._vp = ctypes.c_void_p
        self._torch = torch
        self._buf = torch.zeros(512 * 256 * 8, device=dev, dtype=torch.float16)  # room for 512 markers

    def mark(self, label):
        i = len(self.labels)
        n = (i + 1) * 256 * 8  # i + 1 workgroups of 256 lanes, one 16-byte vector per lane
        if n > self._buf.numel():
            raise RuntimeError("too many trace markers")
        p = self._vp(self._buf.data_ptr())
        sp = self._vp(self._torch.cuda.current_stream().cuda_stream)
        assert self._lib.msd_quick_gelu(p, p, n, self._code, sp) == 0
        self._torch.cuda.synchronize()
        self.labels.append(label)


def _gn_plan_text(msd, batch, channels, hw, elt, in_place=False):
    """'slices per unit x lanes x vectors per lane' of the GroupNorm launch for this shape (output
    apart from the input unless in_place), ', w writers' when w workgroups share each whole unit
    and store a w-th of it each."""
    split, threads, k, writers = msd.groupnorm_plan(batch, channels, hw, 32,
                                                    msd.DTYPE_F16 if elt == 2 else msd.DTYPE_F32,
                                                    in_place=in_place)
    if split == 0:
        return "general kernel"
    text = "%d x %d lanes x %d vectors" % (split, threads, k)
    return text + (", %d writers" % writers if writers > 1 else "")


def _kernel_case(torch, msd, dev, kind, p, dt, batch, sigma=1.0):
    """Buffers, launch closures and byte counts for one row of the per-kernel tables; inputs are
    N(0, sigma).  `launch(x, y, stream)` writes y apart from x; GroupNorm is also timed with
    y == x (launch(x, x, stream)), the form of the reference's out-norms (M/nn/ResBlock.cpp:222)."""
    import ctypes
    vp = ctypes.c_void_p
    lib = msd.load_library()
    code, elt = (msd.DTYPE_F16, 2) if dt == torch.float16 else (msd.DTYPE_F32, 4)
    if kind == "groupnorm_silu":
        n_in = n_out = batch * p["c"] * p["hw"]
        nbytes = 2 * n_in * elt
    elif kind == "layernorm":
        n_in = n_out = p["rows"] * p["dim"]
        nbytes = 2 * n_in * elt
    elif kind == "geglu":
        n_in, n_out = 2 * p["rows"] * p["inner"], p["rows"] * p["inner"]
        nbytes = 3 * n_out * elt
    else:  # elementwise activation
        n_in = n_out = p["n"]
        nbytes = 2 * n_in * elt
    copies = max(4, min(256, int(640e6 // max(nbytes, 1)) + 1))
    xs = [(torch.randn(n_in, device=dev, dtype=torch.float32) * sigma).to(dt) for _ in range(copies)]
    ys = [torch.empty(n_out, device=dev, dtype=dt) for _ in range(copies)]
    cdim = p.get("c", p.get("dim", 1))
    ga = torch.ones(cdim, device=dev)
    be = torch.zeros(cdim, device=dev)

    def launch(x, y, sp):
        if kind == "groupnorm_silu":
            return lib.msd_groupnorm(vp(x.data_ptr()), vp(y.data_ptr()), vp(ga.data_ptr()), vp(be.data_ptr()),
                                     batch, p["c"], p["hw"], 32, 1e-5, 1, code, sp)
        if kind == "layernorm":
            return lib.msd_layernorm(vp(x.data_ptr()), vp(y.data_ptr()), vp(ga.data_ptr()), vp(be.data_ptr()),
                                     p["rows"], p["dim"], 1e-5, code, sp)
        if kind == "geglu":
            return lib.msd_geglu(vp(x.data_ptr()), vp(y.data_ptr()), p["rows"], p["inner"], code, sp)
        return getattr(lib, "msd_" + kind)(vp(x.data_ptr()), vp(y.data_ptr()), p["n"], code, sp)

    copy_dst = {}
    if kind == "geglu":  # a copy of the same traffic reads and writes 1.5 outputs' worth: it needs longer targets
        copy_dst = {x.data_ptr(): torch.empty(nbytes // 2 // elt, device=dev, dtype=dt) for x in xs}

    def copy_launch(x, y, sp):  # the same bytes through the plain copy kernel (half read, half written)
        dst = copy_dst.get(x.data_ptr(), y)
        return lib.msd_copy(vp(x.data_ptr()), vp(dst.data_ptr()), nbytes // 2, sp)
    return {"xs": xs, "ys": ys, "keep": (ga, be, copy_dst), "launch": launch, "copy_launch": copy_launch,
            "bytes": nbytes, "copy_same_bytes": True, "elt": elt}


def shape_cases(torch):
    """(config, kernel, shape, dtype, batch, sigma of the N(0, sigma) input) of the per-kernel
    table: the shapes of BASELINE configs 1 - 4 (config 2 draws x from N(0, 2))."""
    f16, f32 = torch.float16, torch.float32
    cases = [("cfg1", "groupnorm_silu", {"c": 320, "hw": 4096}, f32, 1, 1.0)]
    for c, side in [(320, 64), (640, 32), (1280, 16), (1280, 8), (960, 32), (1920, 16)]:
        cases.append(("cfg2", "groupnorm_silu", {"c": c, "hw": side * side}, f16, BATCH, 2.0))
        cases.append(("cfg2", "groupnorm_silu", {"c": c, "hw": side * side}, f32, BATCH, 2.0))
    for r, d in [(8192, 320), (2048, 640), (512, 1280)]:
        cases.append(("cfg3", "layernorm", {"rows": r, "dim": d}, f16, BATCH, 1.0))
    for r, i in [(8192, 1280), (2048, 2560), (512, 5120)]:
        cases.append(("cfg3", "geglu", {"rows": r, "inner": i}, f16, BATCH, 1.0))
    cases.append(("cfg4", "layernorm", {"rows": 77, "dim": 768}, f32, 1, 1.0))
    cases.append(("cfg4", "layernorm", {"rows": 154, "dim": 768}, f32, 2, 1.0))
    cases.append(("cfg4", "quick_gelu", {"n": 2 * 77 * 3072}, f32, 2, 1.0))
    return cases


def shape_table(torch, msd, dev, stream, floor_us, markers=None):
    """Per-kernel µs / GB/s / % of HBM peak at the shapes of BASELINE configs 1 - 4, each launch
    on its own buffers (rotating over > 600 MB so nothing is cache-resident), graph-replayed.
    Config 2 / 3 at batch 2 in fp16 (GroupNorm also fp32); config 1 (one fp32 tensor) and config 4
    (text-encoder shapes, fp32) are a few hundred KB to 10 MB per launch and are bound by the
    launch floor, not by bandwidth.

    Three yardsticks stand beside every row: `copy_us`, this library's plain 16-byte copy kernel
    over the same bytes; `memcpy_us`, the HIP runtime's own device-to-device copy of the same
    bytes (hipMemcpyDtoDAsync, captured as memcpy nodes and replayed like everything else);
    `floor_model_us` = the launch floor of a graph node + bytes / 8 TB/s.  GroupNorm rows carry
    `us` / `plan` for an output apart from the input and `us_in_place` / `plan_in_place` for
    y == x (the reference's out-norms, M/nn/ResBlock.cpp:222, where no two workgroups may share a
    unit).  `frac_hbm_peak*` = bytes / time / 8 TB/s."""
    import ctypes
    vp = ctypes.c_void_p
    rt = hip_runtime()
    rows = []

    def mark(row, what):
        if markers is not None:
            markers.mark({"row": len(rows), "what": what, "kernel": row["kernel"], "shape": row["shape"],
                          "dtype": row["dtype"], "bytes": row["bytes"]})

    for cfg, kind, p, dt, batch, sigma in shape_cases(torch):
        case = _kernel_case(torch, msd, dev, kind, p, dt, batch, sigma)
        nbytes = case["bytes"]
        row = {"config": cfg, "kernel": kind, "shape": dict(p, batch=batch), "dtype": "f16" if case["elt"] == 2 else "f32",
               "bytes": nbytes}
        mark(row, "us")
        us = _rotating_launch_us(torch, msd, stream, case["launch"], case["xs"], case["ys"])
        gbs = nbytes / us / 1e3
        row.update({"us": round(us, 3), "GBps": round(gbs, 1), "pct_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 1),
                    "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)})
        if kind == "groupnorm_silu":
            row["plan"] = _gn_plan_text(msd, batch, p["c"], p["hw"], case["elt"])
            mark(row, "us_in_place")
            ius = _rotating_launch_us(torch, msd, stream, lambda x, y, sp: case["launch"](x, x, sp), case["xs"],
                                      case["ys"])
            row["us_in_place"] = round(ius, 3)
            row["frac_hbm_peak_in_place"] = round(nbytes / ius / 1e3 / HBM_PEAK_GBS, 4)
            row["plan_in_place"] = _gn_plan_text(msd, batch, p["c"], p["hw"], case["elt"], in_place=True)
        mark(row, "copy_us")
        cus = _rotating_launch_us(torch, msd, stream, case["copy_launch"], case["xs"], case["ys"])
        row["copy_us"] = round(cus, 3)
        row["pct_of_copy_rate"] = round(100.0 * cus / us, 1)
        copy_dst = case["keep"][2]

        def memcpy_launch(x, y, sp):  # the runtime's own copy of the same bytes (half read, half written)
            dst = copy_dst.get(x.data_ptr(), y)
            return rt.hipMemcpyDtoDAsync(vp(dst.data_ptr()), vp(x.data_ptr()), nbytes // 2, sp)
        mark(row, "memcpy_us")
        mus = _rotating_launch_us(torch, msd, stream, memcpy_launch, case["xs"], case["ys"])
        row["memcpy_us"] = round(mus, 3)
        row["pct_of_memcpy_rate"] = round(100.0 * mus / us, 1)
        row["floor_model_us"] = round(floor_us + nbytes / HBM_PEAK_GBS / 1e3, 3)
        if "us_in_place" in row:
            row["pct_of_copy_rate_in_place"] = round(100.0 * cus / row["us_in_place"], 1)
            row["pct_of_memcpy_rate_in_place"] = round(100.0 * mus / row["us_in_place"], 1)
        if cfg in ("cfg1", "cfg4"):
            row["note"] = "launch-bound: %.2f us at 8 TB/s" % (nbytes / HBM_PEAK_GBS / 1e3)
        rows.append(row)
        del case, copy_dst
        torch.cuda.empty_cache()
    return rows


def launch_floor_us(torch, msd, dev, stream):
    """(µs per launch, µs per graph launch): what one more kernel in a captured step costs when
    it moves nothing, and what launching a graph costs whatever it holds.  Chains of 128 and 512
    16-byte copies are replayed as graphs; the first figure is the slope between the two chain
    lengths, the second the remainder of the shorter chain."""
    import ctypes
    vp = ctypes.c_void_p
    lib = msd.load_library()
    xs = [torch.zeros(4, device=dev) for _ in range(512)]
    ys = [torch.zeros(4, device=dev) for _ in range(512)]

    def chain(nodes):
        return nodes * _rotating_launch_us(torch, msd, stream,
                                           lambda x, y, sp: lib.msd_copy(vp(x.data_ptr()), vp(y.data_ptr()), 16, sp),
                                           xs[:nodes], ys[:nodes], budget=40000)
    short, long_ = chain(128), chain(512)
    per_launch = (long_ - short) / 384.0
    return per_launch, max(0.0, short - 128 * per_launch)


def gn_split_table(torch, msd, dev, stream):
    """GroupNorm+SiLU at the config-2 shapes with the launch plan forced: workgroups per
    (sample, group) in {1, 2, 4, 8} x workgroup size in {512, 1024}, next to the automatic
    plan, all with one writer per unit (what a call in place gets: slices with an exchange).
    `auto_vs_best` > 1.03 would mean the plan in groupnorm.hip picks a slow variant.  `writers`
    is the automatic plan of a call whose output lies apart from its input (several workgroups
    share each whole unit), which is how this table's buffers are laid out."""
    lib = msd.load_library()
    rows = []
    for c, side in [(320, 64), (640, 32), (1280, 16), (1280, 8), (960, 32), (1920, 16)]:
        for dt in (torch.float16, torch.float32):
            case = _kernel_case(torch, msd, dev, "groupnorm_silu", {"c": c, "hw": side * side}, dt, BATCH, 2.0)
            times = {}
            try:
                assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, 0) == 0
                writers_us = round(_rotating_launch_us(torch, msd, stream, case["launch"], case["xs"], case["ys"],
                                                       budget=1000), 3)
                assert lib.msd_set_tuning(msd.TUNE_GN_WRITERS, 1) == 0
                code = msd.DTYPE_F16 if case["elt"] == 2 else msd.DTYPE_F32
                for split in (0, 1, 2, 4, 8):
                    for threads in ((0,) if split == 0 else (512, 1024)):
                        assert lib.msd_set_tuning(msd.TUNE_GN_SPLIT, split) == 0
                        assert lib.msd_set_tuning(msd.TUNE_GN_THREADS, threads) == 0
                        plan = msd.groupnorm_plan(BATCH, c, side * side, 32, code, in_place=True)
                        if split and (plan[0] != split or plan[1] != threads):
                            continue  # (the launch cannot follow this setting: slices too short, registers)
                        key = "auto" if split == 0 else "s%d_t%d" % (split, threads)
                        times[key] = round(_rotating_launch_us(torch, msd, stream, case["launch"], case["xs"],
                                                               case["ys"], budget=1000), 3)
            finally:
                lib.msd_set_tuning(msd.TUNE_GN_SPLIT, 0)
                lib.msd_set_tuning(msd.TUNE_GN_THREADS, 0)
                lib.msd_set_tuning(msd.TUNE_GN_WRITERS, 0)
            best = min(v for k, v in times.items() if k != "auto")
            rows.append({"shape": {"c": c, "hw": side * side, "batch": BATCH}, "dtype": "f16" if case["elt"] == 2 else "f32",
                         "us": times, "best_forced_us": best, "auto_vs_best": round(times["auto"] / best, 3),
                         "writers_us": writers_us, "writers_plan": _gn_plan_text(msd, BATCH, c, side * side, case["elt"]),
                         "writers_vs_auto": round(writers_us / times["auto"], 3)})
            del case
            torch.cuda.empty_cache()
    return rows


def unet_gn_shapes():
    """The distinct (channels, side) of the GroupNorms of one UNet step (in- and out-norms of the 22
    ResBlocks; the final norm repeats one of them): 14 shapes."""
    seen = []
    for cin, cout, side in RESBLOCKS:
        for c in (cin, cout):
            if (c, side) not in seen:
                seen.append((c, side))
    return sorted(seen, key=lambda cs: (cs[0] * cs[1] * cs[1], cs[0]))


SWEEP_THREADS = (256, 384, 512, 640, 768, 960, 1024)


def gn_plan_sweep(torch, msd, dev, stream, batches, progress=None):
    """GroupNorm+SiLU at the 14 GroupNorm shapes of the UNet x {fp16, fp32} x `batches` x {in place,
    output apart}: the automatic launch plan timed against every plan the knobs can force
    (1 / 2 / 4 / 8 slices per unit x 256 ... 1024 lanes, and for an output apart from the input also
    2 / 4 / 8 writers per whole unit x the same workgroup sizes).  A forced setting counts only if
    msd_groupnorm_plan confirms that the launch follows it; identical plans are timed once.  The
    automatic plan and the fastest forced one are then timed twice more, alternating, and
    `auto_vs_best` is the ratio of the medians: above 1.03 the planner picked a slow variant.  `rule`
    / `rule_vs_best`: the same for the planning rule alone, with the table of measured plans (which the
    automatic plan consults first) switched off."""
    lib = msd.load_library()
    knobs = (msd.TUNE_GN_SPLIT, msd.TUNE_GN_THREADS, msd.TUNE_GN_WRITERS)

    def set_knobs(split, threads, writers):
        for knob, value in zip(knobs, (split, threads, writers)):
            assert lib.msd_set_tuning(knob, value) == 0

    def text(plan):
        return "%dx%dx%d" % plan[:3] + (" w%d" % plan[3] if plan[3] > 1 else "")

    rows = []
    for batch in batches:
        for c, side in unet_gn_shapes():
            hw = side * side
            for dt, code, elt in ((torch.float16, msd.DTYPE_F16, 2), (torch.float32, msd.DTYPE_F32, 4)):
                case = _kernel_case(torch, msd, dev, "groupnorm_silu", {"c": c, "hw": hw}, dt, batch, 2.0)
                budget = int(min(3000, max(300, 20000.0 / max(3.0, case["bytes"] / 4e6))))
                for in_place in (True, False):
                    launch = (lambda x, y, sp: case["launch"](x, x, sp)) if in_place else case["launch"]

                    def timed():
                        return _rotating_launch_us(torch, msd, stream, launch, case["xs"], case["ys"], budget=budget)
                    try:
                        set_knobs(0, 0, 0)
                        auto_plan = msd.groupnorm_plan(batch, c, hw, 32, code, in_place=in_place)
                        times = {auto_plan: timed()}
                        # the rule alone (the table of measured plans switched off)
                        assert lib.msd_set_tuning(msd.TUNE_GN_PLAN_RULE_ONLY, 1) == 0
                        rule_plan = msd.groupnorm_plan(batch, c, hw, 32, code, in_place=in_place)
                        if rule_plan not in times:
                            times[rule_plan] = timed()
                        assert lib.msd_set_tuning(msd.TUNE_GN_PLAN_RULE_ONLY, 0) == 0
                        for writers in ((1,) if in_place else (1, 2, 4, 8)):
                            for split in ((1, 2, 4, 8) if writers == 1 else (1,)):
                                for threads in SWEEP_THREADS:
                                    set_knobs(split, threads, writers)
                                    plan = msd.groupnorm_plan(batch, c, hw, 32, code, in_place=in_place)
                                    if plan in times or plan[0] != split or plan[1] != threads or plan[3] != writers:
                                        continue
                                    times[plan] = timed()
                        best_plan = min((pl for pl in times if pl != auto_plan), key=lambda pl: times[pl],
                                        default=auto_plan)
                        auto_runs, best_runs = [times[auto_plan]], [times[best_plan]]
                        if best_plan != auto_plan:
                            for _ in range(2):
                                set_knobs(0, 0, 0)
                                auto_runs.append(timed())
                                set_knobs(best_plan[0], best_plan[1], best_plan[3])
                                best_runs.append(timed())
                    finally:
                        set_knobs(0, 0, 0)
                        lib.msd_set_tuning(msd.TUNE_GN_PLAN_RULE_ONLY, 0)
                    auto_us, best_us = sorted(auto_runs)[len(auto_runs) // 2], sorted(best_runs)[len(best_runs) // 2]
                    row = {"batch": batch, "c": c, "hw": hw, "dtype": "f16" if elt == 2 else "f32",
                           "vectors_per_unit": c // 32 * hw * elt // 16, "units": batch * 32,
                           "in_place": in_place, "auto": text(auto_plan), "auto_us": round(auto_us, 3),
                           "best": text(best_plan), "best_us": round(best_us, 3),
                           "auto_vs_best": round(auto_us / best_us, 3),
                           "rule": text(rule_plan), "rule_us": round(times[rule_plan], 3),
                           "rule_vs_best": round(times[rule_plan] / min(best_us, times[rule_plan]), 3),
                           "variants": {text(pl): round(us, 3) for pl, us in sorted(times.items())}}
                    rows.append(row)
                    if progress is not None:
                        progress(row)
                del case
                torch.cuda.empty_cache()
    return rows


def sweep_summary(paths):
    """Markdown summary of gn_plan_sweep rows read from JSON files (bench.py's output line or a
    list of rows): per batch and call form the worst and median auto_vs_best, then every row whose
    automatic plan is more than 3 % behind the fastest forced one."""
    rows = []
    for path in paths:
        with open(path) as f:
            for line in f:
                line = line.strip()
                if not line.startswith(("{", "[")):
                    continue
                data = json.loads(line)
                rows += data["gn_plan_sweep"] if isinstance(data, dict) else data
    out = ["| batch | call | rows | median auto / best | worst auto / best | worst row | rule alone: median | worst | rows > 1.03 |",
           "|---:|---|---:|---:|---:|---|---:|---:|---:|"]
    for batch in sorted(set(r["batch"] for r in rows)):
        for in_place in (True, False):
            sel = [r for r in rows if r["batch"] == batch and r["in_place"] == in_place]
            if not sel:
                continue
            ratios = sorted(r["auto_vs_best"] for r in sel)
            worst = max(sel, key=lambda r: r["auto_vs_best"])
            rule = sorted(r.get("rule_vs_best", float("nan")) for r in sel)
            out.append("| %d | %s | %d | %.3f | %.3f | %d@%d %s: %s %.2f us, %s %.2f us | %.3f | %.3f | %d |" % (
                batch, "in place" if in_place else "apart", len(sel), ratios[len(ratios) // 2], ratios[-1],
                worst["c"], worst["hw"], worst["dtype"], worst["auto"], worst["auto_us"], worst["best"], worst["best_us"],
                rule[len(rule) // 2], rule[-1], sum(1 for v in rule if v > 1.03)))
    slow = [r for r in rows if r["auto_vs_best"] > 1.03]
    out += ["", "Rows with the automatic plan more than 3 %% behind the fastest forced plan: %d of %d." % (len(slow), len(rows))]
    if slow:
        out += ["", "| batch | shape | dtype | call | automatic plan | us | fastest forced plan | us | ratio |",
                "|---:|---|---|---|---|---:|---|---:|---:|"]
        for r in sorted(slow, key=lambda r: -r["auto_vs_best"]):
            out.append("| %d | %d@%d | %s | %s | %s | %.2f | %s | %.2f | %.3f |" % (
                r["batch"], r["c"], r["hw"], r["dtype"], "in place" if r["in_place"] else "apart", r["auto"], r["auto_us"],
                r["best"], r["best_us"], r["auto_vs_best"]))
    return "\n".join(out)


def trace_summary(trace_csv, bench_json, plain_json=None):
    """Markdown table: the rows of the `shapes` table of a profiled bench.py run next to the
    device durations rocprofv3 --kernel-trace recorded for them.  The run's trace is cut at the
    marker launches (TraceMarkers) whose labels the bench line carries in `trace_markers`; inside
    a cut the kernel with the most dispatches is the measured one (the warm-up and the timed
    replays), of which the median begin-to-end duration is reported per (kernel, grid, workgroup)."""
    import csv
    bench = None
    with open(bench_json) as f:
        for line in f:
            if line.startswith("{"):
                bench = json.loads(line)
    labels = bench["trace_markers"]
    disp = []
    with open(trace_csv) as f:
        for r in csv.DictReader(f):
            disp.append((int(r["Start_Timestamp"]), int(r["End_Timestamp"]), r["Kernel_Name"],
                         int(r["Grid_Size_X"]), int(r["Workgroup_Size_X"])))
    disp.sort()
    cuts, current = {}, None
    for start, end, name, grid, wg in disp:
        if "OpQuickGelu" in name and "__half" in name:
            current = grid // 256 - 1
            cuts[current] = []
        elif current is not None:
            cuts[current].append((name, grid, wg, end - start))

    def short(name):
        name = name.replace("msd::(anonymous namespace)::", "").replace("void ", "")
        depth = 0
        for i, ch in enumerate(name):
            depth += ch == "<"
            depth -= ch == ">"
            if ch == "(" and depth == 0:
                return name[:i]
        return name

    rows = bench["shapes"]
    plain = None  # the same table from a run without the profiler, when given
    if plain_json:
        with open(plain_json) as f:
            for line in f:
                if line.startswith("{"):
                    plain = json.loads(line)["shapes"]
    out = ["| config | kernel | shape | dtype | measurement | bytes | bench.py us per launch, graph chain: unprofiled run | this profiled run | "
           "profiled kernel | workgroups x lanes | dispatches | median device us | GB/s at that | frac of 8 TB/s |",
           "|---|---|---|---|---|---:|---:|---:|---|---|---:|---:|---:|---:|"]
    for i, lab in enumerate(labels):
        found = cuts.get(i, [])
        if not found:  # (the runtime's memcpy shows up here only when it runs as a kernel)
            continue
        groups = {}
        for name, grid, wg, dur in found:
            groups.setdefault((name, grid, wg), []).append(dur)
        (name, grid, wg), durs = max(groups.items(), key=lambda kv: len(kv[1]))
        durs.sort()
        med = durs[len(durs) // 2] / 1e3
        row = rows[lab["row"]]
        shape = " ".join("%s=%s" % kv for kv in row["shape"].items())
        gbs = lab["bytes"] / med / 1e3
        same = plain[lab["row"]] if plain and plain[lab["row"]]["shape"] == row["shape"] and plain[lab["row"]]["kernel"] == row["kernel"] \
            else None
        out.append("| %s | %s | %s | %s | %s | %d | %s | %.2f | `%s` | %d x %d | %d | %.2f | %.0f | %.3f |" % (
            row["config"], row["kernel"], shape, row["dtype"], lab["what"], lab["bytes"],
            "%.2f" % same[lab["what"]] if same else "", row[lab["what"]], short(name),
            grid // wg, wg, len(durs), med, gbs, gbs / HBM_PEAK_GBS))
    return "\n".join(out)


def fusion_table(torch, msd, dev, stream):
    """The additions / permute the reference runs next to its norms, as separate launches and
    folded into the norm kernel (fp16, batch 2, graph-replayed on rotating cold buffers)."""
    import ctypes
    vp = ctypes.c_void_p
    lib = msd.load_library()
    F16 = msd.DTYPE_F16
    rows = []

    def measure(bodies, copies):
        out = {}
        for name, fn in bodies.items():
            replay = capture(torch, msd, stream, fn)
            with torch.cuda.stream(stream):
                replay()
                reps = max(2, int(1500 // copies))
                out[name] = event_time_ms(torch, replay, reps) * 1e3 / (reps * copies)
        return out

    def sp():
        return vp(torch.cuda.current_stream().cuda_stream)

    for c, side in [(320, 64), (640, 32), (1280, 16), (1280, 8)]:
        hw = side * side
        n = BATCH * c * hw
        copies = max(4, min(128, int(400e6 // (4 * n)) + 1))
        xs = [torch.randn(n, device=dev).half() for _ in range(copies)]
        ys = [torch.empty(n, device=dev, dtype=torch.float16) for _ in range(copies)]
        emb = torch.randn(BATCH * c, device=dev).half()
        ga, be = torch.ones(c, device=dev), torch.zeros(c, device=dev)
        g, b, e = vp(ga.data_ptr()), vp(be.data_ptr()), vp(emb.data_ptr())

        def add_then_norm():
            for x in xs:
                xp = vp(x.data_ptr())
                assert lib.msd_chunkwise_add(xp, e, xp, n, hw, F16, sp()) == 0
                assert lib.msd_groupnorm(xp, xp, g, b, BATCH, c, hw, 32, 1e-5, 1, F16, sp()) == 0

        def add_norm_fused():
            for x in xs:
                xp = vp(x.data_ptr())
                assert lib.msd_chunk_add_groupnorm(xp, e, xp, g, b, BATCH, c, hw, 32, 1e-5, 1, F16, sp()) == 0

        def norm_then_permute():
            for x, y in zip(xs, ys):
                xp, yp = vp(x.data_ptr()), vp(y.data_ptr())
                assert lib.msd_groupnorm(xp, xp, g, b, BATCH, c, hw, 32, 1e-6, 0, F16, sp()) == 0
                assert lib.msd_permute_0_2_1(xp, yp, BATCH, c, hw, F16, sp()) == 0

        def norm_tokens_fused():
            for x, y in zip(xs, ys):
                assert lib.msd_groupnorm_tokens(vp(x.data_ptr()), vp(y.data_ptr()), g, b, BATCH, c, hw, 32,
                                                1e-6, F16, sp()) == 0

        t = measure({"a2": add_then_norm, "a1": add_norm_fused, "p2": norm_then_permute,
                     "p1": norm_tokens_fused}, copies)
        rows.append({"what": "chunkwise_add + GroupNorm+SiLU (ResBlock out-norm)", "shape": {"c": c, "hw": hw},
                     "us_separate": round(t["a2"], 2), "us_fused": round(t["a1"], 2),
                     "speedup": round(t["a2"] / t["a1"], 2)})
        rows.append({"what": "GroupNorm + permute to tokens (SpatialTransformer)", "shape": {"c": c, "hw": hw},
                     "us_separate": round(t["p2"], 2), "us_fused": round(t["p1"], 2),
                     "speedup": round(t["p2"] / t["p1"], 2)})
        del xs, ys
    for r, d in [(8192, 320), (2048, 640), (512, 1280)]:
        n = r * d
        copies = max(4, min(128, int(400e6 // (8 * n)) + 1))
        xs = [torch.randn(n, device=dev).half() for _ in range(copies)]
        rs = [torch.randn(n, device=dev).half() for _ in range(copies)]
        ys = [torch.empty(n, device=dev, dtype=torch.float16) for _ in range(copies)]
        ga, be = torch.ones(d, device=dev), torch.zeros(d, device=dev)
        g, b = vp(ga.data_ptr()), vp(be.data_ptr())

        def add_then_ln():
            for x, res, y in zip(xs, rs, ys):
                xp, rp, yp = vp(x.data_ptr()), vp(res.data_ptr()), vp(y.data_ptr())
                assert lib.msd_elemwise_add(xp, rp, xp, n, F16, sp()) == 0
                assert lib.msd_layernorm(xp, yp, g, b, r, d, 1e-5, F16, sp()) == 0

        def add_ln_fused():
            for x, res, y in zip(xs, rs, ys):
                xp, rp, yp = vp(x.data_ptr()), vp(res.data_ptr()), vp(y.data_ptr())
                assert lib.msd_add_layernorm(xp, rp, xp, yp, g, b, r, d, 1e-5, F16, sp()) == 0

        t = measure({"l2": add_then_ln, "l1": add_ln_fused}, copies)
        rows.append({"what": "elemwise_add + LayerNorm (transformer block)", "shape": {"rows": r, "dim": d},
                     "us_separate": round(t["l2"], 2), "us_fused": round(t["l1"], 2),
                     "speedup": round(t["l2"] / t["l1"], 2)})
        del xs, rs, ys
    torch.cuda.empty_cache()
    return rows


def neighbour_table(torch, msd, dev, stream):
    """The kernels either side of the path: attention row softmax (fp16, in place) next to a
    plain copy of the same bytes, the Linear layers on the time-embedding rows with the SiLU
    folded in or launched separately, the stand-alone permute next to a copy, and the DDIM latent
    update (graph-replayed)."""
    import ctypes
    vp = ctypes.c_void_p
    lib = msd.load_library()
    F16, F32 = msd.DTYPE_F16, msd.DTYPE_F32
    rows = []

    def sp():
        return vp(torch.cuda.current_stream().cuda_stream)

    def measure(fn, launches, budget=1500):
        replay = capture(torch, msd, stream, fn)
        with torch.cuda.stream(stream):
            replay()
            reps = max(2, int(budget // launches))
            return event_time_ms(torch, replay, reps) * 1e3 / (reps * launches)

    # softmax over keys: self-attention of the three UNet levels (batch 2 x 8 heads) and the
    # cross-attention against 77 text tokens
    for r, c in [(2 * 8 * 4096, 4096), (2 * 8 * 1024, 1024), (2 * 8 * 256, 256), (2 * 8 * 4096, 77),
                 (2 * 8 * 1024, 77)]:
        nbytes = 2 * r * c * 2
        copies = max(2, min(64, int(1.2e9 // nbytes) + 1))
        xs = [(torch.randn(r * c, device=dev) * 2.0).half() for _ in range(copies)]
        ys = [torch.empty(r * c, device=dev, dtype=torch.float16) for _ in range(2)]

        def body():
            for x in xs:
                assert lib.msd_softmax(vp(x.data_ptr()), vp(x.data_ptr()), r, c, 0, F16, sp()) == 0

        def copy_body():
            for i, x in enumerate(xs):
                assert lib.msd_copy(vp(x.data_ptr()), vp(ys[i % 2].data_ptr()), r * c * 2, sp()) == 0
        us, cus = measure(body, copies, 400), measure(copy_body, copies, 400)
        gbs = nbytes / us / 1e3
        rows.append({"kernel": "softmax", "shape": {"rows": r, "cols": c}, "dtype": "f16", "bytes": nbytes,
                     "us": round(us, 2), "GBps": round(gbs, 1), "pct_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 1),
                     "copy_us": round(cus, 2), "pct_of_copy_rate": round(100 * cus / us, 1)})
        del xs, ys
        torch.cuda.empty_cache()

    # Linear on the two embedding rows; 16 weight sets in rotation (never cache-resident together
    # with their predecessors at 1280 x 1280 fp32 = 6.5 MB each)
    for n, k, what in [(1280, 320, "time_embed_0 + SiLU"), (1280, 1280, "time_embed_2"),
                       (1280, 1280, "SiLU(emb) + embed_linear"), (320, 1280, "SiLU(emb) + embed_linear")]:
        for dt, code, elt in ((torch.float16, F16, 2), (torch.float32, F32, 4)):
            copies = 16
            ws = [(torch.randn(n, k, device=dev) * k ** -0.5).to(dt) for _ in range(copies)]
            bias = torch.zeros(n, device=dev)
            x = torch.randn(BATCH, k, device=dev).to(dt)
            tmp = torch.empty_like(x)
            y = torch.empty(BATCH, n, device=dev, dtype=dt)
            act_in = 1 if what.startswith("SiLU") else 0
            act_out = 1 if what.endswith("SiLU") else 0

            def fused():
                for w in ws:
                    assert lib.msd_linear_rows(vp(x.data_ptr()), vp(w.data_ptr()), vp(bias.data_ptr()),
                                               vp(y.data_ptr()), BATCH, n, k, act_in, act_out, code, sp()) == 0

            def separate():
                for w in ws:
                    src = x
                    if act_in:
                        assert lib.msd_silu(vp(x.data_ptr()), vp(tmp.data_ptr()), BATCH * k, code, sp()) == 0
                        src = tmp
                    assert lib.msd_linear_rows(vp(src.data_ptr()), vp(w.data_ptr()), vp(bias.data_ptr()),
                                               vp(y.data_ptr()), BATCH, n, k, 0, 0, code, sp()) == 0
                    if act_out:
                        assert lib.msd_silu(vp(y.data_ptr()), vp(y.data_ptr()), BATCH * n, code, sp()) == 0
            us = measure(fused, copies)
            row = {"kernel": "linear_rows", "what": what, "shape": {"m": BATCH, "n": n, "k": k},
                   "dtype": "f16" if elt == 2 else "f32", "bytes": n * k * elt, "us": round(us, 2),
                   "GBps": round(n * k * elt / us / 1e3, 1)}
            if act_in or act_out:
                row["us_separate_silu"] = round(measure(separate, copies), 2)
            rows.append(row)
            del ws

    # the 22 per-ResBlock SiLU(emb) -> Linear(1280 -> Cout) projections of one step: 22 launches
    # against one grouped launch (4 weight sets in rotation, 52 MB each in fp16)
    couts = [c for _, c, _ in RESBLOCKS]
    for dt, code, elt in ((torch.float16, F16, 2), (torch.float32, F32, 4)):
        sets = 4
        ws = [[(torch.randn(n, 1280, device=dev) * 1280 ** -0.5).to(dt) for n in couts] for _ in range(sets)]
        bs = [torch.zeros(n, device=dev) for n in couts]
        ys = [torch.empty(BATCH, n, device=dev, dtype=dt) for n in couts]
        x = torch.randn(BATCH, 1280, device=dev).to(dt)
        cnt = len(couts)
        tables = []
        for wset in ws:
            tables.append(((vp * cnt)(*[w.data_ptr() for w in wset]), (vp * cnt)(*[b.data_ptr() for b in bs]),
                           (vp * cnt)(*[y.data_ptr() for y in ys]), (ctypes.c_size_t * cnt)(*couts)))

        def separate22():
            for wset in ws:
                for w, b, y, n in zip(wset, bs, ys, couts):
                    assert lib.msd_linear_rows(vp(x.data_ptr()), vp(w.data_ptr()), vp(b.data_ptr()), vp(y.data_ptr()),
                                               BATCH, n, 1280, 1, 0, code, sp()) == 0

        def grouped22():
            for wp, bp, yp, ns in tables:
                assert lib.msd_linear_rows_grouped(vp(x.data_ptr()), wp, bp, yp, ns, cnt, BATCH, 1280, 1, 0, code,
                                                   sp()) == 0
        us_sep = measure(separate22, sets, 200)
        us_grp = measure(grouped22, sets, 200)
        nbytes = sum(couts) * 1280 * elt
        rows.append({"kernel": "linear_rows_grouped", "what": "22 x SiLU(emb) + embed_linear of one UNet step",
                     "shape": {"m": BATCH, "k": 1280, "n_total": sum(couts)}, "dtype": "f16" if elt == 2 else "f32",
                     "bytes": nbytes, "us": round(us_grp, 2), "GBps": round(nbytes / us_grp / 1e3, 1),
                     "us_22_launches": round(us_sep, 2), "speedup": round(us_sep / us_grp, 2)})
        del ws, tables
        torch.cuda.empty_cache()

    # tokens -> NCHW behind a SpatialTransformer (the permute that stays a launch of its own), next
    # to a plain copy of the same bytes
    for tokens, dim in [(4096, 320), (1024, 640), (256, 1280)]:
        count = BATCH * tokens * dim
        nbytes = 2 * count * 2
        copies = max(4, min(32, int(300e6 // nbytes)))
        xs = [torch.randn(count, device=dev).half() for _ in range(copies)]
        ys = [torch.empty(count, device=dev, dtype=torch.float16) for _ in range(copies)]
        us = _rotating_launch_us(torch, msd, stream, lambda x, y, s_: lib.msd_permute_0_2_1(
            vp(x.data_ptr()), vp(y.data_ptr()), BATCH, tokens, dim, F16, s_), xs, ys, budget=600)
        cus = _rotating_launch_us(torch, msd, stream, lambda x, y, s_: lib.msd_copy(
            vp(x.data_ptr()), vp(y.data_ptr()), count * 2, s_), xs, ys, budget=600)
        gbs = nbytes / us / 1e3
        rows.append({"kernel": "permute_0_2_1", "shape": {"i": BATCH, "j": tokens, "k": dim}, "dtype": "f16",
                     "bytes": nbytes, "us": round(us, 2), "GBps": round(gbs, 1),
                     "pct_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 1), "copy_us": round(cus, 2),
                     "pct_of_copy_rate": round(100 * cus / us, 1)})
        del xs, ys
        torch.cuda.empty_cache()

    # DDIM update of the latent, batch 2 x [4, 64, 64] float32, in place
    n = BATCH * 4 * 64 * 64
    x, e = torch.randn(n, device=dev), torch.randn(n, device=dev)

    def ddim_body():
        for _ in range(16):
            assert lib.msd_ddim_update(vp(x.data_ptr()), vp(e.data_ptr()), vp(x.data_ptr()), n, 0.5, 0.6,
                                       0.70710678, F32, sp()) == 0
    rows.append({"kernel": "ddim_update", "shape": {"n": n}, "dtype": "f32", "bytes": 3 * n * 4,
                 "us": round(measure(ddim_body, 16), 2)})
    torch.cuda.empty_cache()
    return rows


def large_batch_table(torch, msd, dev, stream):
    """The same kernels on tensors 16 times larger than the UNet step's (batch 32), where the
    launch floor no longer matters: what each kernel sustains against a plain copy."""
    import ctypes
    vp = ctypes.c_void_p
    lib = msd.load_library()
    rt = hip_runtime()
    F16 = msd.DTYPE_F16
    B = 32
    rows = []

    def sp():
        return vp(torch.cuda.current_stream().cuda_stream)

    def measure(fn, launches):
        replay = capture(torch, msd, stream, fn)
        with torch.cuda.stream(stream):
            # the GPU has idled while the buffers were made: replay for some tens of milliseconds
            # first so that the clocks are back up when the timed batches start
            t0 = time.perf_counter()
            while time.perf_counter() - t0 < 0.05:
                for _ in range(10):
                    replay()
                torch.cuda.synchronize()
            reps = max(10, 240 // launches)
            return event_time_ms(torch, replay, reps) * 1e3 / (reps * launches)

    cases = [("groupnorm_silu", {"batch": B, "c": 320, "hw": 4096}, B * 320 * 4096, B * 320 * 4096),
             ("groupnorm_silu", {"batch": B, "c": 640, "hw": 1024}, B * 640 * 1024, B * 640 * 1024),
             ("groupnorm_silu", {"batch": B, "c": 1280, "hw": 256}, B * 1280 * 256, B * 1280 * 256),
             ("layernorm", {"rows": B * 4096, "dim": 320}, B * 4096 * 320, B * 4096 * 320),
             ("geglu", {"rows": B * 4096, "inner": 1280}, B * 4096 * 2560, B * 4096 * 1280)]
    for kind, p, n_in, n_out in cases:
        copies = max(3, int(1.0e9 // (2 * (n_in + n_out))))  # rotate over about a gigabyte: nothing stays cached
        xs = [torch.randn(n_in, device=dev).half() for _ in range(copies)]
        ys = [torch.empty(n_out, device=dev, dtype=torch.float16) for _ in range(copies)]
        d = p.get("c", p.get("dim", 1))
        ga, be = torch.ones(d, device=dev), torch.zeros(d, device=dev)

        def body():
            for x, y in zip(xs, ys):
                if kind == "groupnorm_silu":
                    rc = lib.msd_groupnorm(vp(x.data_ptr()), vp(y.data_ptr()), vp(ga.data_ptr()), vp(be.data_ptr()),
                                           B, p["c"], p["hw"], 32, 1e-5, 1, F16, sp())
                elif kind == "layernorm":
                    rc = lib.msd_layernorm(vp(x.data_ptr()), vp(y.data_ptr()), vp(ga.data_ptr()), vp(be.data_ptr()),
                                           p["rows"], p["dim"], 1e-5, F16, sp())
                else:
                    rc = lib.msd_geglu(vp(x.data_ptr()), vp(y.data_ptr()), p["rows"], p["inner"], F16, sp())
                assert rc == 0

        def copy_body():  # the same total bytes: read half, write half
            for x, y in zip(xs, ys):
                assert lib.msd_copy(vp(x.data_ptr()), vp(y.data_ptr()), 2 * n_out, sp()) == 0

        def memcpy_body():  # the same through the HIP runtime's own device-to-device copy
            for x, y in zip(xs, ys):
                assert rt.hipMemcpyDtoDAsync(vp(y.data_ptr()), vp(x.data_ptr()), 2 * n_out, sp()) == 0
        nbytes = 2 * (n_in + n_out)
        us = measure(body, copies)
        row = {"kernel": kind, "shape": p, "dtype": "f16", "bytes": nbytes, "us": round(us, 2),
               "GBps": round(nbytes / us / 1e3, 1), "pct_hbm_peak": round(100 * nbytes / us / 1e3 / HBM_PEAK_GBS, 1)}
        if n_in == n_out:
            cus = measure(copy_body, copies)
            row["copy_us"] = round(cus, 2)
            row["pct_of_copy_rate"] = round(100 * cus / us, 1)
            mus = measure(memcpy_body, copies)
            row["memcpy_us"] = round(mus, 2)
            row["pct_of_memcpy_rate"] = round(100 * mus / us, 1)
        if kind == "groupnorm_silu":
            row["plan"] = _gn_plan_text(msd, B, p["c"], p["hw"], 2)
        rows.append(row)
        del xs, ys
        torch.cuda.empty_cache()
    return rows


def step_with_adds(torch, msd, dev, stream):
    """One UNet step of the path including the additions the reference runs right before its
    norms (the embedding add before each ResBlock out-norm, the residual add before LayerNorm 2
    and 3 of each transformer block): as separate launches in the reference's order, and
    folded into the norm kernels.  Same buffers, graph-replayed.

    A second pair adds the Linear layers on the embedding rows that the reference runs between
    those launches (time_embed_0 / SiLU / time_embed_2, M/UNetModel.cpp:1107-1120, and SiLU(emb)
    -> embed_linear in every ResBlock, M/nn/ResBlock.cpp:173-183, whose output is what the
    embedding add adds): every launch separate, against SiLU folded into the Linear kernels and
    the 22 projections as ONE grouped launch ahead of the blocks.

    A third pair adds the 16 SpatialTransformer norms (GroupNorm without SiLU, then the permute to
    tokens, M/nn/SpatialTransformer.cpp:127-139) as two launches each, against the one launch of
    msd_groupnorm_tokens."""
    import ctypes
    vp = ctypes.c_void_p
    lib = msd.load_library()
    F16 = msd.DTYPE_F16
    g = torch.Generator(device=dev).manual_seed(77)
    keep = []

    def randn(*shape, dtype=torch.float16):
        t = torch.randn(*shape, device=dev, dtype=torch.float32, generator=g).to(dtype)
        keep.append(t)
        return t

    affine = {}

    def gb(c):
        if c not in affine:
            affine[c] = (1.0 + 0.1 * randn(c, dtype=torch.float32), 0.1 * randn(c, dtype=torch.float32))
        return affine[c]

    separate, fused = [], []  # lists of (fn, args)
    separate_emb, fused_emb = [], []  # the same with the embedding-row Linear layers
    st_separate, st_fused = [], []    # the SpatialTransformer norms: GroupNorm + permute against one launch
    # embedding path: sinusoid [2, 320] -> h [2, 1280] -> emb [2, 1280] -> per ResBlock [2, Cout]
    couts = [c for _, c, _ in RESBLOCKS]
    temb_out = torch.empty((BATCH, 320), device=dev, dtype=torch.float16)
    h_buf = torch.empty((BATCH, 1280), device=dev, dtype=torch.float16)
    emb_buf = torch.empty((BATCH, 1280), device=dev, dtype=torch.float16)
    emb_act = torch.empty((BATCH, 1280), device=dev, dtype=torch.float16)
    w_te0, w_te2 = randn(1280, 320) * 320 ** -0.5, randn(1280, 1280) * 1280 ** -0.5
    w_res = [randn(c, 1280) * 1280 ** -0.5 for c in couts]
    b_te = 0.1 * randn(1280, dtype=torch.float32)
    b_res = [0.1 * randn(c, dtype=torch.float32) for c in couts]
    proj = [torch.empty((BATCH, c), device=dev, dtype=torch.float16) for c in couts]
    keep += [temb_out, h_buf, emb_buf, emb_act, w_te0, w_te2, b_te] + w_res + b_res + proj
    cnt = len(couts)
    group_tables = ((vp * cnt)(*[w.data_ptr() for w in w_res]), (vp * cnt)(*[b.data_ptr() for b in b_res]),
                    (vp * cnt)(*[y.data_ptr() for y in proj]), (ctypes.c_size_t * cnt)(*couts))
    keep.append(group_tables)

    def lin(x, w, b, y, n, k, act_in, act_out):
        return (lib.msd_linear_rows, (vp(x.data_ptr()), vp(w.data_ptr()), vp(b.data_ptr()), vp(y.data_ptr()), BATCH, n, k,
                                      act_in, act_out, F16))
    out_norm, ln_count, res_index = False, 0, -1
    for kind, p in step_layers():
        if kind == "temb":
            t = torch.randint(0, 1000, (BATCH,), device=dev, dtype=torch.int64, generator=g)
            keep += [t]
            call = (lib.msd_timestep_embedding, (vp(t.data_ptr()), vp(temb_out.data_ptr()), BATCH, p["dim"], 10000.0, F16))
            for lst in (separate, fused, separate_emb, fused_emb):
                lst.append(call)
        elif kind == "silu":
            x = randn(p["n"])
            call = (lib.msd_silu, (vp(x.data_ptr()), vp(x.data_ptr()), p["n"], F16))
            separate.append(call), fused.append(call)
            if res_index < 0:  # the time-embedding MLP: Linear, SiLU, Linear
                separate_emb.append(lin(temb_out, w_te0, b_te, h_buf, 1280, 320, 0, 0))
                separate_emb.append((lib.msd_silu, (vp(h_buf.data_ptr()), vp(h_buf.data_ptr()), BATCH * 1280, F16)))
                separate_emb.append(lin(h_buf, w_te2, b_te, emb_buf, 1280, 1280, 0, 0))
                fused_emb.append(lin(temb_out, w_te0, b_te, h_buf, 1280, 320, 0, 1))
                fused_emb.append(lin(h_buf, w_te2, b_te, emb_buf, 1280, 1280, 0, 0))
                fused_emb.append((lib.msd_linear_rows_grouped, (vp(emb_buf.data_ptr()),) + group_tables +
                                  (cnt, BATCH, 1280, 1, 0, F16)))
            else:              # a ResBlock's SiLU(emb) -> embed_linear (already done by the grouped launch)
                separate_emb.append((lib.msd_silu, (vp(emb_buf.data_ptr()), vp(emb_act.data_ptr()), BATCH * 1280, F16)))
                separate_emb.append(lin(emb_act, w_res[res_index], b_res[res_index], proj[res_index], couts[res_index],
                                        1280, 0, 0))
            res_index += 1
            out_norm = True  # the next GroupNorm is the ResBlock's out-norm (after the embedding add)
        elif kind == "gn_silu":
            c, hw = p["c"], p["hw"]
            x = randn(BATCH, c, hw) * 2.0
            keep.append(x)
            y = x if p["inplace"] else torch.empty_like(x)
            keep.append(y)
            ga, be = gb(c)
            xp, yp = vp(x.data_ptr()), vp(y.data_ptr())
            gp, bp = vp(ga.data_ptr()), vp(be.data_ptr())
            if out_norm and p["inplace"]:
                emb = randn(BATCH * c)
                ep = vp(emb.data_ptr())
                separate.append((lib.msd_chunkwise_add, (xp, ep, xp, BATCH * c * hw, hw, F16)))
                separate.append((lib.msd_groupnorm, (xp, yp, gp, bp, BATCH, c, hw, 32, 1e-5, 1, F16)))
                fused.append((lib.msd_chunk_add_groupnorm, (xp, ep, yp, gp, bp, BATCH, c, hw, 32, 1e-5, 1, F16)))
                pp = vp(proj[res_index - 1].data_ptr())  # this ResBlock's projection of the embedding
                assert couts[res_index - 1] == c
                separate_emb.append((lib.msd_chunkwise_add, (xp, pp, xp, BATCH * c * hw, hw, F16)))
                separate_emb.append((lib.msd_groupnorm, (xp, yp, gp, bp, BATCH, c, hw, 32, 1e-5, 1, F16)))
                fused_emb.append((lib.msd_chunk_add_groupnorm, (xp, pp, yp, gp, bp, BATCH, c, hw, 32, 1e-5, 1, F16)))
                out_norm = False
            else:
                call = (lib.msd_groupnorm, (xp, yp, gp, bp, BATCH, c, hw, 32, 1e-5, 1, F16))
                for lst in (separate, fused, separate_emb, fused_emb):
                    lst.append(call)
        elif kind == "ln":
            rows, dim = p["rows"], p["dim"]
            x, y = randn(rows, dim), torch.empty((rows, dim), device=dev, dtype=torch.float16)
            keep.append(y)
            ga, be = gb(dim)
            xp, yp, gp, bp = vp(x.data_ptr()), vp(y.data_ptr()), vp(ga.data_ptr()), vp(be.data_ptr())
            if ln_count % 3 == 0:  # LayerNorm 1 of a block has no add in front
                # the SpatialTransformer's own norm ahead of the block (M/nn/SpatialTransformer.cpp:127-139):
                # GroupNorm(eps 1e-6, no SiLU) over [B, dim, tokens], then the permute to [B, tokens, dim]
                sx = randn(BATCH, dim, rows // BATCH) * 2.0
                sy, sz = torch.empty_like(sx), torch.empty_like(sx)
                keep.extend([sy, sz])
                sga, sbe = gb(dim)
                sxp, syp, szp = vp(sx.data_ptr()), vp(sy.data_ptr()), vp(sz.data_ptr())
                st_separate.append((lib.msd_groupnorm, (sxp, syp, vp(sga.data_ptr()), vp(sbe.data_ptr()), BATCH, dim,
                                                        rows // BATCH, 32, 1e-6, 0, F16)))
                st_separate.append((lib.msd_permute_0_2_1, (syp, szp, BATCH, dim, rows // BATCH, F16)))
                st_fused.append((lib.msd_groupnorm_tokens, (sxp, szp, vp(sga.data_ptr()), vp(sbe.data_ptr()), BATCH, dim,
                                                            rows // BATCH, 32, 1e-6, F16)))
                call = (lib.msd_layernorm, (xp, yp, gp, bp, rows, dim, 1e-5, F16))
                for lst in (separate, fused, separate_emb, fused_emb):
                    lst.append(call)
            else:
                res = randn(rows, dim)
                rp = vp(res.data_ptr())
                for lst in (separate, separate_emb):
                    lst.append((lib.msd_elemwise_add, (xp, rp, xp, rows * dim, F16)))
                    lst.append((lib.msd_layernorm, (xp, yp, gp, bp, rows, dim, 1e-5, F16)))
                for lst in (fused, fused_emb):
                    lst.append((lib.msd_add_layernorm, (xp, rp, xp, yp, gp, bp, rows, dim, 1e-5, F16)))
            ln_count += 1
        else:
            rows, inner = p["rows"], p["inner"]
            x = randn(rows, 2 * inner)
            y = torch.empty((rows, inner), device=dev, dtype=torch.float16)
            keep.append(y)
            call = (lib.msd_geglu, (vp(x.data_ptr()), vp(y.data_ptr()), rows, inner, F16))
            for lst in (separate, fused, separate_emb, fused_emb):
                lst.append(call)

    def runner(calls):
        def run():
            sp = vp(torch.cuda.current_stream().cuda_stream)
            for fn, args in calls:
                assert fn(*args, sp) == 0
        return run

    out = {}
    separate_all, fused_all = separate_emb + st_separate, fused_emb + st_fused
    for name, calls in (("separate", separate), ("fused", fused), ("separate_emb", separate_emb),
                        ("fused_emb", fused_emb), ("separate_all", separate_all), ("fused_all", fused_all)):
        replay = capture(torch, msd, stream, runner(calls))
        with torch.cuda.stream(stream):
            for _ in range(5):
                replay()
            out[name] = event_time_ms(torch, replay, 50) / 50
    return {"launches_separate": len(separate), "launches_fused": len(fused),
            "ms_separate": round(out["separate"], 4), "ms_fused": round(out["fused"], 4),
            "speedup": round(out["separate"] / out["fused"], 3),
            "with_embedding_linears": {
                "launches_separate": len(separate_emb), "launches_fused_grouped": len(fused_emb),
                "ms_separate": round(out["separate_emb"], 4), "ms_fused_grouped": round(out["fused_emb"], 4),
                "speedup": round(out["separate_emb"] / out["fused_emb"], 3)},
            "with_spatial_transformer_norms_too": {
                "launches_separate": len(separate_all), "launches_fused": len(fused_all),
                "ms_separate": round(out["separate_all"], 4), "ms_fused": round(out["fused_all"], 4),
                "speedup": round(out["separate_all"] / out["fused_all"], 3)}}


def cpu_baseline(total_bytes, budget_s=24.0):
    """The reference path as host loops (the CPU oracle, fp32, unfused passes exactly as the
    reference enqueues them) over the layers of one full step, timed on this host's cores.
    Every layer runs `reps` times on its own input (reps sized so the whole leg takes about
    `budget_s` seconds of CPU work); the figure is per step."""
    import numpy as np
    from oracle import pyoracle as orc
    threads = orc.max_threads()

    def run(kind, p, data):
        if kind == "gn_silu":
            orc.groupnorm(data[0], data[1], data[2], 32, 1e-5, silu=True)
        elif kind == "ln":
            orc.layernorm(data[0], data[1], data[2], 1e-5)
        elif kind == "geglu":
            orc.geglu(data[0])
        elif kind == "silu":
            orc.silu(data[0])
        else:
            for t in (17, 801):
                orc.timestep_embedding(t)

    def make(kind, p):
        if kind == "gn_silu":
            return (orc.normal((BATCH, p["c"], p["hw"]), seed=p["c"] + p["hw"], sigma=2.0),
                    np.ones(p["c"], np.float32), np.zeros(p["c"], np.float32))
        if kind == "ln":
            return (orc.normal((p["rows"], p["dim"]), seed=p["rows"] + p["dim"]),
                    np.ones(p["dim"], np.float32), np.zeros(p["dim"], np.float32))
        if kind == "geglu":
            return (orc.normal((p["rows"], 2 * p["inner"]), seed=p["rows"] + p["inner"]),)
        if kind == "silu":
            return (orc.normal((p["n"],), seed=1),)
        return ()

    layers = step_layers()

    def timed_pass(reps):
        total = 0.0
        for kind, p in layers:
            data = make(kind, p)
            t0 = time.perf_counter()
            for _ in range(reps):
                run(kind, p, data)
            total += time.perf_counter() - t0
        return total

    probe = timed_pass(1)  # also warms the thread pool; sizes the timed pass
    reps = max(2, min(400, int(budget_s / max(probe, 1e-3))))
    t_total = timed_pass(reps)
    per_step = t_total / reps
    return {"value": round(total_bytes / per_step / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "ms_per_step": round(per_step * 1e3, 2), "seconds_timed": round(t_total, 2),
            "sample": "the layers of one full UNet step (45 GN+SiLU, 48 LN, 16 GEGLU, 23 SiLU, 1 embedding), "
                      "%d repetitions each, fp32, unfused passes as the reference enqueues them, OpenMP over "
                      "groups/rows; GB/s uses the same fp16 algorithmic bytes as the GPU figure; oracle built "
                      "with %s" % (reps, orc.build_flags())}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--mode", choices=["graph", "eager"], default="graph")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-shapes", action="store_true", help="skip the per-kernel tables")
    ap.add_argument("--tables", default="shapes,gn_split,fusions,neighbours,large_batch",
                    help="comma list of the per-kernel tables to measure (also: gn_plan_sweep, the automatic "
                         "GroupNorm launch plan against every forced one at --sweep-batches; minutes per batch)")
    ap.add_argument("--sweep-batches", default="1,2,4,8,16,32", help="batches of the gn_plan_sweep table")
    ap.add_argument("--sweep-summary", default=None, metavar="JSON[,JSON...]",
                    help="no GPU: print the markdown summary of gn_plan_sweep rows in these bench.py outputs")
    ap.add_argument("--trace-summary", default=None, metavar="KERNEL_TRACE_CSV",
                    help="no GPU: print the `shapes` rows of --bench-json next to the device durations in this "
                         "rocprofv3 --kernel-trace CSV of the same run")
    ap.add_argument("--bench-json", default=None, help="the bench.py output (file) of the profiled run")
    ap.add_argument("--plain-json", default=None, help="a bench.py output of a run without the profiler, for comparison")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="for rocprofv3 --pmc runs: one 64 MiB device copy (known traffic) then three "
                         "eager steps; prints nothing")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no cross-GPU step and the build uses a single "
              "device; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.sweep_summary:
        print(sweep_summary(args.sweep_summary.split(",")))
        return
    if args.trace_summary:
        print(trace_summary(args.trace_summary, args.bench_json, args.plain_json))
        return

    import ctypes
    import torch
    msd = importlib.import_module("mobile-stable-diffusion_amd")
    msd.load_library()  # raises if the HIP library is not built
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.Stream()
    step = Step(msd, torch, dev)

    if args.pmc_probe:
        a = torch.empty(64 << 20, dtype=torch.uint8, device=dev)
        b = torch.empty_like(a)
        a.random_(0, 255)
        torch.cuda.synchronize()
        for _ in range(3):
            b.copy_(a)  # plain copy kernel: reads 64 MiB, writes 64 MiB
        torch.cuda.synchronize()
        msd.init()
        for _ in range(3):
            step.run(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        assert msd.status() == 0
        return

    def eager_step():
        step.run(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))

    with torch.cuda.stream(stream):
        if args.mode == "graph":
            run_step = capture(torch, msd, stream, eager_step)
        else:
            msd.init()
            run_step = eager_step
        for _ in range(args.warmup):
            run_step()
        seconds = timed_replays(torch, run_step, args.steps)
        assert msd.status() == 0
        ms_per_step = seconds * 1e3 / args.steps
        value = step.bytes / (seconds / args.steps) / 1e9

        # the same launches as plain copies of the same bytes: the ceiling of this launch structure
        copy_step = CopyStep(msd, torch, dev)

        def eager_copy_step():
            copy_step.run(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        run_copy = capture(torch, msd, stream, eager_copy_step) if args.mode == "graph" else eager_copy_step
        for _ in range(max(3, args.warmup // 4)):
            run_copy()
        copy_reps = max(10, args.steps // 4)
        copy_ms = timed_replays(torch, run_copy, copy_reps) * 1e3 / copy_reps
        del copy_step

        # the same step with the 23 norms the reference runs in place (ResBlock out-norms, final norm)
        # given output buffers of their own: several workgroups can then share every unit
        apart_step = Step(msd, torch, dev, norms_in_place=False)

        def eager_apart_step():
            apart_step.run(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        run_apart = capture(torch, msd, stream, eager_apart_step) if args.mode == "graph" else eager_apart_step
        for _ in range(max(3, args.warmup // 4)):
            run_apart()
        apart_ms = timed_replays(torch, run_apart, copy_reps) * 1e3 / copy_reps
        del apart_step

        # per-kernel-family timing inside the same step order (HIP events on the launch stream)
        families = {}
        for kind in ("gn_silu", "ln", "geglu"):
            def fam(kind=kind):
                step.run(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream), only=kind)
            replay = capture(torch, msd, stream, fam) if args.mode == "graph" else fam
            for _ in range(3):
                replay()
            reps = max(5, args.steps // 4)
            ms = event_time_ms(torch, replay, reps) / reps
            k = step.by_kind[kind]
            gbs = k["bytes"] / ms / 1e6
            families[kind] = {"launches": k["launches"], "bytes": k["bytes"], "us_total": round(ms * 1e3, 2),
                              "us_per_launch": round(ms * 1e3 / k["launches"], 3), "GBps": round(gbs, 1),
                              "pct_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 1)}

    # One block per kernel family: algorithmic bytes per launch / live HIP-event time per launch
    # against the 8 TB/s peak, with the HBM traffic per launch that rocprofv3 --pmc FETCH_SIZE /
    # WRITE_SIZE measured (profiles/traffic.json).  The top level of `roofline` is the single kernel
    # with the largest total GPU time in the rocprofv3 kernel statistics of this workload,
    # geglu_kernel<__half, 1>; the GroupNorm family as a whole takes more of the step and sits
    # furthest below the roofline, which `roofline.families` shows.
    traffic = measured_traffic()
    kernel_names = {"gn_silu": "gn_slice_kernel<__half, K, true, SHARED>", "ln": "ln_team_kernel<__half, NW, VPL, TL, EARLY>",
                    "geglu": "geglu_kernel<__half, 1>"}
    roofline_families = {}
    for kind, fam in families.items():
        roofline_families[kind] = {
            "bound": "hbm", "kernel": kernel_names[kind], "achieved": fam["GBps"], "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": round(fam["GBps"] / HBM_PEAK_GBS, 4), "launches_per_step": fam["launches"],
            "bytes_per_launch": fam["bytes"] // fam["launches"], "us_per_launch": fam["us_per_launch"],
            "pct_of_step_time": round(100 * fam["us_total"] / (ms_per_step * 1e3), 1),
            "traffic": traffic.get(kind)}
    roofline = dict(roofline_families["geglu"])
    roofline["families"] = roofline_families

    out = {
        "metric": "fused GroupNorm+SiLU/LayerNorm/GEGLU HBM GB/s over one SD UNet step (batch 2, fp16 storage)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "unet_step_norm_act: 45 GroupNorm(32)+SiLU, 48 LayerNorm, 16 GEGLU, 23 SiLU(emb), "
                               "1 timestep embedding at SD UNet shapes, batch 2, fp16 storage / fp32 arithmetic",
                   "bytes_per_step": step.bytes, "launches_per_step": len(step.launches), "launch_mode": args.mode,
                   "pct_hbm_peak": round(100 * value / HBM_PEAK_GBS, 1),
                   "copy_step_ms": round(copy_ms, 4), "pct_of_copy_step_rate": round(100 * copy_ms / ms_per_step, 1),
                   "ms_per_step_all_norms_out_of_place": round(apart_ms, 4)},
        "roofline": roofline,
        "kernel_families": families,
    }
    floor_us, graph_us = launch_floor_us(torch, msd, dev, stream)
    out["config"]["launch_floor_us"] = round(floor_us, 3)
    out["config"]["graph_launch_us"] = round(graph_us, 2)
    tables = set() if args.no_shapes else set(t for t in args.tables.split(",") if t)
    if "shapes" in tables:
        markers = TraceMarkers(torch, msd, dev)
        out["shapes"] = shape_table(torch, msd, dev, stream, floor_us, markers)
        out["trace_markers"] = markers.labels
    if "gn_split" in tables:
        out["gn_split"] = gn_split_table(torch, msd, dev, stream)
    if "fusions" in tables:
        out["fusions"] = fusion_table(torch, msd, dev, stream)
    if "fusions" in tables:
        out["step_with_adds"] = step_with_adds(torch, msd, dev, stream)
    if "large_batch" in tables:
        out["large_batch"] = large_batch_table(torch, msd, dev, stream)
    if "neighbours" in tables:
        out["neighbours"] = neighbour_table(torch, msd, dev, stream)
    if "gn_plan_sweep" in tables:
        def progress(row):  # a long table: one line per row on stderr keeps the run visibly alive
            print("gn_plan_sweep batch %d %d@%d %s %s: auto %s %.2f us, best %s %.2f us" % (
                row["batch"], row["c"], row["hw"], row["dtype"], "in place" if row["in_place"] else "apart",
                row["auto"], row["auto_us"], row["best"], row["best_us"]), file=sys.stderr, flush=True)
        out["gn_plan_sweep"] = gn_plan_sweep(torch, msd, dev, stream, [int(b) for b in args.sweep_batches.split(",") if b],
                                             progress)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(step.bytes)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
