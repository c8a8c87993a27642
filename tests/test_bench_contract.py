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
