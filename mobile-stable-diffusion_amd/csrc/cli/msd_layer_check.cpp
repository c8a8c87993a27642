// msd_layer_check: runs layer objects the way the reference's own in-source tests do --
// construct from .npy weight names, init(), forward(), then util::testBuffer against a
// golden .npy (the commented checks at M/nn/ResBlock.cpp:129-133,
// M/nn/BasicTransformerBlock.cpp:119-161) -- for every case listed in a manifest, using
// only the public C++ headers.  One line per case, file names relative to the media path:
//
//   groupnorm  <channels> <groups> <eps> <batch> <silu 0|1> <f32|f16> <weight> <bias> <input> <golden>
//   layernorm  <dim> <eps> <f32|f16> <weight> <bias> <input> <golden>
//   geglu      <in_features> <out_features> <f32|f16> <projected> <golden>
//   linear     <in_features> <out_features> <silu_in 0|1> <silu_out 0|1> <f32|f16> <weight> <bias|-> <input> <golden>
//   softmax    <chunk> <stable 0|1> <f32|f16> <input> <golden>
//
//   msd_layer_check MEDIA_DIR MANIFEST [--rel 1e-5] [--abs16 2e-3]
//
// A case passes when the buffer has the golden's size and max |diff| <= rel * max(1, |golden|)
// bound (float32 storage; the per-element check is done here, testBuffer prints the summary)
// or <= abs16 (float16 storage).  Exit status: number of failed cases (0 = all passed), 100 for
// usage / file errors.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <exception>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

#include "Activation.h"
#include "GEGLU.h"
#include "GroupNorm.h"
#include "LayerNorm.h"
#include "Linear.h"
#include "util.h"

using namespace msd;

namespace {

double g_rel = 1e-5, g_abs16 = 2e-3;

DType parse_dtype(const std::string &s) {
    if (s == "f32") return DType::F32;
    if (s == "f16") return DType::F16;
    throw std::runtime_error("storage type must be f32 or f16, got " + s);
}

// true when `out` matches the golden file under the criterion of its storage type
bool verdict(hipStream_t stream, const DeviceBuffer &out, const std::string &golden) {
    const util::TestResult r = util::testBuffer(stream, out, golden.c_str());  // prints the summary line
    if (!r.size_matches) return false;
    const std::vector<float> got = util::download(out, stream);
    const npy::Array want = util::load_npy_file(golden);
    for (size_t i = 0; i < got.size(); i++) {
        const double d = std::fabs((double)got[i] - (double)want.data[i]);
        const double bound = out.dtype() == DType::F16
                                 ? std::fmax(g_abs16, std::ldexp(1.0, std::ilogb(std::fmax(std::fabs((double)want.data[i]), 6.2e-5)) - 10))
                                 : g_rel * std::fmax(1.0, std::fabs((double)want.data[i]));
        if (!(d <= bound)) {
            fprintf(stderr, "  element %zu: %f vs %f exceeds %g\n", i, got[i], want.data[i], bound);
            return false;
        }
    }
    return true;
}

bool run_case(hipStream_t stream, const std::string &line) {
    std::istringstream in(line);
    std::string kind;
    in >> kind;
    if (kind == "groupnorm") {
        size_t channels, groups, batch;
        float eps;
        int silu;
        std::string dt, w, b, x, golden;
        in >> channels >> groups >> eps >> batch >> silu >> dt >> w >> b >> x >> golden;
        GroupNorm layer(stream, groups, channels, eps, w, b, batch, silu != 0);
        layer.init();
        DeviceBuffer input = util::upload(util::load_npy_file(x).data, parse_dtype(dt), stream);
        DeviceBuffer output = DeviceBuffer::allocate(input.bytes(), input.dtype());
        if (layer.forward(input, output) != 0) return false;
        return verdict(stream, output, golden);
    }
    if (kind == "layernorm") {
        size_t dim;
        float eps;
        std::string dt, w, b, x, golden;
        in >> dim >> eps >> dt >> w >> b >> x >> golden;
        LayerNorm layer(stream, dim, w, b, eps);
        layer.init();
        DeviceBuffer input = util::upload(util::load_npy_file(x).data, parse_dtype(dt), stream);
        DeviceBuffer output = DeviceBuffer::allocate(input.bytes(), input.dtype());
        if (layer.forward(input, output) != 0) return false;
        return verdict(stream, output, golden);
    }
    if (kind == "geglu") {
        size_t in_features, out_features;
        std::string dt, x, golden;
        in >> in_features >> out_features >> dt >> x >> golden;
        GEGLU layer(stream, in_features, out_features);
        layer.init();
        DeviceBuffer input = util::upload(util::load_npy_file(x).data, parse_dtype(dt), stream);
        DeviceBuffer output = DeviceBuffer::allocate(input.bytes() / 2, input.dtype());
        if (layer.forward(input, output) != 0) return false;
        return verdict(stream, output, golden);
    }
    if (kind == "linear") {
        size_t in_features, out_features;
        int silu_in, silu_out;
        std::string dt, w, b, x, golden;
        in >> in_features >> out_features >> silu_in >> silu_out >> dt >> w >> b >> x >> golden;
        Linear layer(stream, in_features, out_features, w, b == "-" ? "" : b, parse_dtype(dt));
        layer.init();
        DeviceBuffer input = util::upload(util::load_npy_file(x).data, parse_dtype(dt), stream);
        const size_t rows = input.count() / in_features;
        DeviceBuffer output = DeviceBuffer::allocate(rows * out_features * dtype_size(input.dtype()), input.dtype());
        if (layer.forwardSilu(input, output, silu_in != 0, silu_out != 0) != 0) return false;
        return verdict(stream, output, golden);
    }
    if (kind == "softmax") {
        size_t chunk;
        int stable;
        std::string dt, x, golden;
        in >> chunk >> stable >> dt >> x >> golden;
        DeviceBuffer buf = util::upload(util::load_npy_file(x).data, parse_dtype(dt), stream);
        if (softmax(stream, buf, buf, chunk, stable != 0) != 0) return false;  // in place, as the reference
        return verdict(stream, buf, golden);
    }
    throw std::runtime_error("unknown case kind: " + kind);
}

}  // namespace

int main(int argc, char **argv) {
    std::vector<std::string> pos;
    for (int i = 1; i < argc; i++) {
        const std::string a = argv[i];
        if ((a == "--rel" || a == "--abs16") && i + 1 < argc) {
            (a == "--rel" ? g_rel : g_abs16) = atof(argv[++i]);
        } else {
            pos.push_back(a);
        }
    }
    if (pos.size() != 2) {
        fprintf(stderr, "usage: msd_layer_check MEDIA_DIR MANIFEST [--rel TOL] [--abs16 TOL]\n");
        return 100;
    }
    util::setMediaPath(pos[0]);
    std::ifstream manifest(pos[1]);
    if (!manifest) {
        fprintf(stderr, "cannot open manifest %s\n", pos[1].c_str());
        return 100;
    }
    hipStream_t stream = nullptr;
    if (hipStreamCreate(&stream) != hipSuccess) {
        fprintf(stderr, "no usable GPU stream\n");
        return 100;
    }
    int failed = 0, total = 0;
    std::string line;
    while (std::getline(manifest, line)) {
        if (line.empty() || line[0] == '#') continue;
        total++;
        bool ok = false;
        try {
            ok = run_case(stream, line);
        } catch (const std::exception &e) {
            fprintf(stderr, "  exception: %s\n", e.what());
        }
        printf("%s  %s\n", ok ? "PASS" : "FAIL", line.c_str());
        fflush(stdout);
        failed += ok ? 0 : 1;
    }
    (void)hipStreamSynchronize(stream);
    (void)hipStreamDestroy(stream);
    printf("%d of %d cases passed\n", total - failed, total);
    return failed > 99 ? 99 : failed;
}
