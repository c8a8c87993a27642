"""Build recipe for the native libraries (hipcc cross-compiles gfx950 without a GPU).

    libmsd_hip.so   HIP kernels + the C ABI declared in include/msd_hip.h
    libmsd_nn.so    C++ host layer objects (GroupNorm / LayerNorm / GEGLU / ...) on top of it
    cli/msd_compare golden-file comparison tool (host only)
    cli/msd_layer_check  runs the layer objects against golden .npy files (needs a GPU)

Run as a script (`python build.py`) or call build_all().
"""
import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
REPO = os.path.dirname(PKG_DIR)

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# -packed-fp32-ops is switched off: plain float code must not be turned into
# v_pk_*_f32 instructions.
DEVICE_FLAGS = [
    "-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]

LIB_HIP = os.path.join(CSRC, "libmsd_hip.so")
LIB_NN = os.path.join(CSRC, "libmsd_nn.so")
CLI_COMPARE = os.path.join(CSRC, "cli", "msd_compare")
CLI_LAYER_CHECK = os.path.join(CSRC, "cli", "msd_layer_check")


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if proc.returncode != 0:
        raise RuntimeError("build failed: %s\n%s" % (" ".join(cmd), out))
    return out


HIP_SOURCES = ["api.hip", "gn_plan.hip", "groupnorm.hip", "layernorm.hip", "stream_ops.hip", "embed_ops.hip"]


def build_hip():
    """Compiles each translation unit to an object (in parallel) and links libmsd_hip.so."""
    from concurrent.futures import ThreadPoolExecutor
    objs = [os.path.join(CSRC, s.replace(".hip", ".o")) for s in HIP_SOURCES]

    def compile_one(pair):
        src, obj = pair
        return _run([HIPCC] + DEVICE_FLAGS + ["-c", "-o", obj, os.path.join(CSRC, src)])

    with ThreadPoolExecutor(max_workers=6) as pool:
        list(pool.map(compile_one, zip(HIP_SOURCES, objs)))
    _run([HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-Wno-unused-command-line-argument",
          "-o", LIB_HIP] + objs)
    return LIB_HIP


def build_nn():
    nn_dir = os.path.join(CSRC, "nn")
    srcs = sorted(os.path.join(nn_dir, f) for f in os.listdir(nn_dir) if f.endswith(".cpp"))
    if not srcs:
        return None
    # host-only C++ against the HIP runtime API: the system compiler, no device code
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared",
           "-D__HIP_PLATFORM_AMD__", "-I", "/opt/rocm/include", "-I", os.path.join(REPO, "include"),
           "-I", nn_dir, "-Wall", "-Wno-deprecated-declarations"] + srcs + [
           "-o", LIB_NN, "-L", CSRC, "-lmsd_hip", "-L/opt/rocm/lib", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,/opt/rocm/lib"]
    _run(cmd)
    return LIB_NN


def build_cli():
    """msd_compare: host-only golden-file comparison tool (no HIP, no GPU)."""
    nn_dir = os.path.join(CSRC, "nn")
    _run([os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-Wall", "-I", nn_dir,
          os.path.join(CSRC, "cli", "msd_compare.cpp"), os.path.join(nn_dir, "npy.cpp"), "-o", CLI_COMPARE])
    return CLI_COMPARE


def build_layer_check():
    """msd_layer_check: the layer objects against golden .npy files, from C++ alone."""
    nn_dir = os.path.join(CSRC, "nn")
    _run([os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-Wall", "-Wno-deprecated-declarations",
          "-D__HIP_PLATFORM_AMD__", "-I", "/opt/rocm/include", "-I", os.path.join(REPO, "include"), "-I", nn_dir,
          os.path.join(CSRC, "cli", "msd_layer_check.cpp"), "-o", CLI_LAYER_CHECK, "-L", CSRC, "-lmsd_nn",
          "-lmsd_hip", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,$ORIGIN/..", "-Wl,-rpath,/opt/rocm/lib"])
    return CLI_LAYER_CHECK


def build_all(verbose=True):
    built = [build_hip()]
    nn = build_nn()
    if nn:
        built.append(nn)
    built.append(build_cli())
    if nn:
        built.append(build_layer_check())
    if verbose:
        for b in built:
            print("built", b)
    return built


if __name__ == "__main__":
    build_all()
    sys.exit(0)
