"""bench.py's workload definition and command line, checked without a GPU: the step is BASELINE
config 5 (one timestep embedding, 23 SiLU on the embedding, 45 GroupNorm+SiLU, 48 LayerNorm,
16 GEGLU at the SD UNet shapes, batch 2, fp16) with the algorithmic bytes that follow from those shapes,
in the reference's order (M/nn/ResBlock.cpp:125-232, M/nn/BasicTransformerBlock.cpp:116-164,
M/UNetModel.cpp:1796-1810), and a run on more than one GPU is refused."""
import os
import subprocess
import sys
from collections import Counter

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_step_is_the_full_unet_step_of_config_5():
    layers = bench.step_layers()
    kinds = Counter(kind for kind, _ in layers)
    assert kinds == {"temb": 1, "silu": 23, "gn_silu": 45, "ln": 48, "geglu": 16}
    assert len(layers) == 133
    by_kind = Counter()
    for kind, p in layers:
        by_kind[kind] += bench.layer_bytes(kind, p)
    # 44 ResBlock norms + the final norm; 48 LayerNorms; 16 GEGLUs (fp16, gamma / beta not counted)
    assert by_kind["gn_silu"] == 257_556_480 + 10_485_760
    assert by_kind["ln"] == 277_217_280
    assert by_kind["geglu"] == 554_434_560
    assert sum(by_kind.values()) == 1_099_694_080
    # the reference's order inside a ResBlock: in-norm (own output), SiLU(emb), out-norm in place
    first = [i for i, (kind, _) in enumerate(layers) if kind == "gn_silu"][0]
    assert [k for k, _ in layers[first:first + 3]] == ["gn_silu", "silu", "gn_silu"]
    assert layers[first][1]["inplace"] is False and layers[first + 2][1]["inplace"] is True
    assert layers[-1] == ("gn_silu", {"c": 320, "hw": 4096, "inplace": True})     # final norm + SiLU
    # every transformer block: three LayerNorms, then GEGLU on 4 * dim
    for i, (kind, p) in enumerate(layers):
        if kind == "geglu":
            assert [k for k, _ in layers[i - 3:i]] == ["ln", "ln", "ln"]
            assert p["inner"] == 4 * layers[i - 1][1]["dim"] and p["rows"] == layers[i - 1][1]["rows"]


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 2
    assert "one GPU" in (r.stdout + r.stderr)


def test_trace_summary_cuts_a_kernel_trace_at_the_marker_launches(tmp_path):
    """bench.py --trace-summary: the dispatches of a rocprofv3 kernel trace are attributed to the
    `shapes` measurement whose marker launch (quick_GELU on fp16, i + 1 workgroups) precedes them,
    the kernel with the most dispatches inside a cut is the measured one, and its median duration
    gives the row's GB/s.  A synthetic trace: two measurements of one row."""
    import json
    bench_line = {
        "shapes": [{"config": "cfg2", "kernel": "groupnorm_silu", "shape": {"c": 320, "hw": 4096, "batch": 2},
                    "dtype": "f16", "bytes": 10485760, "us": 5.2, "us_in_place": 5.9}],
        "trace_markers": [{"row": 0, "what": "us", "bytes": 10485760}, {"row": 0, "what": "us_in_place", "bytes": 10485760}],
    }
    bench_json = tmp_path / "bench.json"
    bench_json.write_text("some log line\n" + json.dumps(bench_line) + "\n")
    marker = "void msd::(anonymous namespace)::act_kernel<__half, msd::(anonymous namespace)::OpQuickGelu, 1>(...)"
    apart = "void msd::(anonymous namespace)::gn_slice_kernel<__half, 5, true, true>(...)"
    in_place = "void msd::(anonymous namespace)::gn_slice_kernel<__half, 2, true, false>(...)"
    rows, t = [], 1000
    def add(name, grid, wg, dur):
        nonlocal t
        rows.append({"Kernel_Name": name, "Start_Timestamp": t, "End_Timestamp": t + dur, "Grid_Size_X": grid,
                     "Workgroup_Size_X": wg})
        t += dur + 500
    add(apart, 256 * 1024, 1024, 9999)              # before the first marker: ignored
    add(marker, 256 * 1, 256, 900)
    for dur in (5000, 5200, 5100, 30000):           # median 5200 ns (even count: the upper middle)
        add(apart, 256 * 1024, 1024, dur)
    add(marker, 256 * 2, 256, 900)
    add(apart, 256 * 1024, 1024, 7000)              # a stray launch of another kernel inside the cut
    for dur in (6000, 6100, 5900):
        add(in_place, 256 * 640, 640, dur)
    trace = tmp_path / "trace.csv"
    cols = ["Kernel_Name", "Start_Timestamp", "End_Timestamp", "Grid_Size_X", "Workgroup_Size_X"]
    trace.write_text(",".join('"%s"' % c for c in cols) + "\n" +
                     "\n".join(",".join('"%s"' % r[c] for c in cols) for r in reversed(rows)) + "\n")  # any order
    text = bench.trace_summary(str(trace), str(bench_json))
    lines = [l for l in text.splitlines() if l.startswith("| cfg2")]
    assert len(lines) == 2
    assert "gn_slice_kernel<__half, 5, true, true>" in lines[0] and "| 256 x 1024 | 4 | 5.20 |" in lines[0]
    assert "| 10485760 |  | 5.20 |" in lines[0]     # no unprofiled run given: that column stays empty
    assert "gn_slice_kernel<__half, 2, true, false>" in lines[1] and "| 256 x 640 | 3 | 6.00 |" in lines[1]
    assert "| %.0f | %.3f |" % (10485760 / 5.2 / 1e3, 10485760 / 5.2 / 1e3 / 8000.0) in lines[0]


def test_sweep_summary_reports_the_worst_row_per_batch(tmp_path):
    import json
    def row(batch, in_place, ratio, rule_ratio):
        return {"batch": batch, "c": 320, "hw": 4096, "dtype": "f16", "in_place": in_place, "auto": "4x640x2",
                "auto_us": 6.0 * ratio, "best": "4x768x2", "best_us": 6.0, "auto_vs_best": ratio, "rule": "2x512x5",
                "rule_us": 6.0 * rule_ratio, "rule_vs_best": rule_ratio, "variants": {}}
    out = tmp_path / "sweep.json"
    out.write_text(json.dumps({"gn_plan_sweep": [row(2, True, 1.01, 1.02), row(2, True, 1.05, 1.08), row(32, False, 0.99, 1.0)]}) + "\n")
    text = bench.sweep_summary([str(out)])
    assert "| 2 | in place | 2 | 1.050 | 1.050 |" in text and "| 1.080 | 1.080 | 1 |" in text
    assert "| 32 | apart | 1 | 0.990 | 0.990 |" in text
    assert "more than 3 % behind the fastest forced plan: 1 of 3." in text
