#include "UNetNormActStep.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <stdexcept>

#include "Activation.h"
#include "util.h"

namespace msd {
namespace {

struct Res {
    size_t cin, cout, side;
    bool transformer;
};

// ResBlocks in execution order: input blocks 1,2,4,5,7,8,10,11, middle (2), output 0..11
const Res kResBlocks[22] = {
    {320, 320, 64, true},    {320, 320, 64, true},    {320, 640, 32, true},   {640, 640, 32, true},
    {640, 1280, 16, true},   {1280, 1280, 16, true},  {1280, 1280, 8, false}, {1280, 1280, 8, false},
    {1280, 1280, 8, true},   {1280, 1280, 8, false},  {2560, 1280, 8, false}, {2560, 1280, 8, false},
    {2560, 1280, 8, false},  {2560, 1280, 16, true},  {2560, 1280, 16, true}, {1920, 1280, 16, true},
    {1920, 640, 32, true},   {1280, 640, 32, true},   {960, 640, 32, true},   {960, 320, 64, true},
    {640, 320, 64, true},    {640, 320, 64, true},
};

// deterministic synthetic values: splitmix64 + Box-Muller
struct Rng {
    uint64_t s;
    uint64_t next() {
        s += 0x9E3779B97F4A7C15ull;
        uint64_t z = s;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    double u01() { return ((double)(next() >> 11) + 0.5) * (1.0 / 9007199254740992.0); }
    float normal() {
        const double r = std::sqrt(-2.0 * std::log(u01()));
        return (float)(r * std::cos(6.283185307179586 * u01()));
    }
};

std::vector<float> normals(Rng &rng, size_t n, float mean, float sigma) {
    std::vector<float> v(n);
    for (float &x : v) x = mean + sigma * rng.normal();
    return v;
}

}  // namespace

UNetNormActStep::UNetNormActStep(hipStream_t stream, size_t batch, DType dtype, unsigned seed, bool keep_inputs)
    : keep_inputs(keep_inputs), stream(stream), batch(batch), dtype(dtype) {
    Rng rng{seed};
    const size_t elt = dtype_size(dtype);
    auto activation = [&](size_t n, float sigma) {
        buffers.push_back(util::upload(normals(rng, n, 0.0f, sigma), dtype, stream));
        return buffers.size() - 1;
    };
    auto blank = [&](size_t n) {
        buffers.push_back(DeviceBuffer::allocate(n * elt, dtype));
        return buffers.size() - 1;
    };
    // a device copy of an input that its layer overwrites, when asked for
    auto keep = [&](size_t in) -> size_t {
        if (!keep_inputs) return npos;
        kept_inputs.push_back(DeviceBuffer::allocate(buffers[in].bytes(), dtype));
        if (hipMemcpyAsync(kept_inputs.back().ptr(), buffers[in].ptr(), buffers[in].bytes(),
                           hipMemcpyDeviceToDevice, stream) != hipSuccess)
            throw std::runtime_error("UNetNormActStep: copy failed");
        return kept_inputs.size() - 1;
    };
    auto add_group_norm = [&](size_t channels, size_t hw, bool in_place) {
        group_norms.emplace_back(new GroupNorm(stream, 32, channels, 1e-5f, "", "", batch, true));
        std::vector<float> g = normals(rng, channels, 1.0f, 0.1f), b = normals(rng, channels, 0.0f, 0.1f);
        group_norms.back()->init(g, b);
        const size_t n = batch * channels * hw;
        const size_t in = activation(n, 2.0f);
        const size_t out = in_place ? in : blank(n);
        ops.push_back({0, group_norms.size() - 1, in, out, {channels, hw}, g, b, in_place ? keep(in) : npos});
        algorithmic_bytes += 2 * n * elt;
    };
    auto add_silu_emb = [&]() {  // SiLU on the [batch, 4*MODEL_CHANNELS] time embedding
        const size_t n = batch * 1280;
        const size_t in = activation(n, 1.0f);
        ops.push_back({3, 0, in, blank(n), {n, 0}, {}, {}, npos});
    };

    timestep_dev = DeviceBuffer::allocate(batch * sizeof(int64_t), DType::F32);
    embedding = DeviceBuffer::allocate(batch * 320 * elt, dtype);
    {
        const size_t n = batch * 1280;  // SiLU inside the time-embedding MLP, in place
        const size_t in = activation(n, 1.0f);
        ops.push_back({3, 0, in, in, {n, 0}, {}, {}, keep(in)});
    }
    for (const Res &r : kResBlocks) {
        const size_t hw = r.side * r.side;
        add_group_norm(r.cin, hw, false);
        add_silu_emb();
        add_group_norm(r.cout, hw, true);
        if (r.transformer) {
            const size_t dim = r.cout, rows = batch * hw;
            for (int i = 0; i < 3; i++) {
                layer_norms.emplace_back(new LayerNorm(stream, dim, "", ""));
                std::vector<float> g = normals(rng, dim, 1.0f, 0.1f), b = normals(rng, dim, 0.0f, 0.1f);
                layer_norms.back()->init(g, b);
                const size_t in = activation(rows * dim, 1.0f);
                ops.push_back({1, layer_norms.size() - 1, in, blank(rows * dim), {rows, dim}, g, b, npos});
                algorithmic_bytes += 2 * rows * dim * elt;
            }
            geglus.emplace_back(new GEGLU(stream, dim, 4 * dim));
            const size_t in = activation(rows * 8 * dim, 1.0f);
            ops.push_back({2, geglus.size() - 1, in, blank(rows * 4 * dim), {rows, 4 * dim}, {}, {}, npos});
            algorithmic_bytes += 3 * rows * 4 * dim * elt;
        }
    }
    add_group_norm(320, 64 * 64, true);  // final norm + SiLU
    if (hipStreamSynchronize(stream) != hipSuccess) throw std::runtime_error("UNetNormActStep: sync failed");
}

UNetNormActStep::~UNetNormActStep() {
    if (graph_exec) (void)hipGraphExecDestroy(graph_exec);
    if (graph) (void)hipGraphDestroy(graph);
}

void UNetNormActStep::setTimesteps(const std::vector<long> &timesteps) {
    if (timesteps.size() != batch) throw std::runtime_error("one timestep per sample expected");
    std::vector<int64_t> host(timesteps.begin(), timesteps.end());
    // ordered behind the work already on the stream (an earlier step may still read the old values)
    hipError_t err = hipStreamSynchronize(stream);
    if (err == hipSuccess)
        err = hipMemcpy(timestep_dev.ptr(), host.data(), batch * sizeof(int64_t), hipMemcpyHostToDevice);
    if (err != hipSuccess)
        throw std::runtime_error(std::string("UNetNormActStep: timestep upload failed: ") + hipGetErrorString(err));
}

int UNetNormActStep::restoreInputs() {
    if (!keep_inputs) throw std::runtime_error("UNetNormActStep was built without keep_inputs");
    for (const Op &op : ops) {
        if (op.kept == npos) continue;
        const hipError_t err = hipMemcpyAsync(buffers[op.in].ptr(), kept_inputs[op.kept].ptr(),
                                              buffers[op.in].bytes(), hipMemcpyDeviceToDevice, stream);
        if (err != hipSuccess) return (int)err;
    }
    return MSD_OK;
}

UNetNormActStep::OpInfo UNetNormActStep::opInfo(size_t i) const {
    const Op &op = ops.at(i);
    return OpInfo{op.kind, {op.dims[0], op.dims[1]}, op.in == op.out};
}

std::vector<float> UNetNormActStep::downloadInput(size_t i) const { return util::download(buffers[ops.at(i).in], stream); }
std::vector<float> UNetNormActStep::downloadOutput(size_t i) const { return util::download(buffers[ops.at(i).out], stream); }
std::vector<float> UNetNormActStep::downloadEmbedding() const { return util::download(embedding, stream); }

int UNetNormActStep::forward(const std::vector<long> &timesteps) {
    setTimesteps(timesteps);
    int rc = msd_timestep_embedding(static_cast<const int64_t *>(timestep_dev.ptr()), embedding.ptr(), batch,
                                    320, 10000.0f, (int)dtype, stream);
    for (size_t i = 0; i < ops.size() && rc == MSD_OK; i++) {
        const Op &op = ops[i];
        switch (op.kind) {
            case 0: rc = group_norms[op.layer]->forward(buffers[op.in], buffers[op.out]); break;
            case 1: rc = layer_norms[op.layer]->forward(buffers[op.in], buffers[op.out]); break;
            case 2: rc = geglus[op.layer]->forward(buffers[op.in], buffers[op.out]); break;
            default: rc = silu(stream, buffers[op.in], buffers[op.out]); break;
        }
    }
    return rc;
}

int UNetNormActStep::forwardGraph() {
    if (!graph_exec) {
        if (stream == nullptr) throw std::runtime_error("graph capture needs a non-default stream");
        hipError_t err = hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal);
        if (err != hipSuccess) return (int)err;
        int rc = msd_timestep_embedding(static_cast<const int64_t *>(timestep_dev.ptr()), embedding.ptr(),
                                        batch, 320, 10000.0f, (int)dtype, stream);
        for (size_t i = 0; i < ops.size() && rc == MSD_OK; i++) {
            const Op &op = ops[i];
            switch (op.kind) {
                case 0: rc = group_norms[op.layer]->forward(buffers[op.in], buffers[op.out]); break;
                case 1: rc = layer_norms[op.layer]->forward(buffers[op.in], buffers[op.out]); break;
                case 2: rc = geglus[op.layer]->forward(buffers[op.in], buffers[op.out]); break;
                default: rc = silu(stream, buffers[op.in], buffers[op.out]); break;
            }
        }
        err = hipStreamEndCapture(stream, &graph);
        if (rc == MSD_OK && err == hipSuccess) err = hipGraphInstantiate(&graph_exec, graph, nullptr, nullptr, 0);
        if (rc != MSD_OK || err != hipSuccess) {  // nothing half-built survives: the next call starts over
            if (graph_exec) (void)hipGraphExecDestroy(graph_exec);
            if (graph) (void)hipGraphDestroy(graph);
            graph_exec = nullptr;
            graph = nullptr;
            return rc != MSD_OK ? rc : (int)err;
        }
    }
    return (int)hipGraphLaunch(graph_exec, stream);
}

}  // namespace msd
