// One UNet step's worth of the norm / activation / embedding path, in the call order of
// UNetModel::forward (M/UNetModel.cpp:1078-1929): the timestep embedding and the SiLU of the
// time-embedding MLP, then for each of the 22 ResBlocks GroupNorm+SiLU (in), SiLU(emb),
// GroupNorm+SiLU (out, in place) (M/nn/ResBlock.cpp:125-142,173-180,222-232), for the 16
// blocks that carry a transformer three LayerNorms and the GEGLU epilogue
// (M/nn/BasicTransformerBlock.cpp:116,136,158; M/nn/FeedForward.cpp:71), and the final
// GroupNorm+SiLU (M/UNetModel.cpp:1796-1810).  Convolutions, GEMMs and attention between
// them are not part of this library, so each layer works on its own synthetic buffers.
// Used to measure the path end to end from C++ (eagerly or as one captured HIP graph).
#pragma once

#include <hip/hip_runtime_api.h>

#include <memory>
#include <vector>

#include "DeviceBuffer.h"
#include "GEGLU.h"
#include "GroupNorm.h"
#include "LayerNorm.h"

namespace msd {

class UNetNormActStep {
public:
    // batch: samples per step (2 = classifier-free guidance); dtype: activation storage.
    // keep_inputs: keep a device copy of every input that a layer overwrites in place, so that
    // restoreInputs() can put it back (for checking the outputs of repeated steps).
    UNetNormActStep(hipStream_t stream, size_t batch, DType dtype, unsigned seed = 5001,
                    bool keep_inputs = false);
    ~UNetNormActStep();

    // Uploads one timestep per sample (the integers of DDIMSampler's list, M/DDIMSampler.cpp:78-82).
    void setTimesteps(const std::vector<long> &timesteps);
    // Enqueues every layer of one step on the stream.  Returns 0 or the first error code.
    int forward(const std::vector<long> &timesteps);
    // Captures the step into a HIP graph once, then replays it; the graph reads the timesteps
    // from device memory, so setTimesteps() between replays takes effect.  Returns 0 or an error code.
    int forwardGraph();
    // Copies the kept inputs back over the buffers that in-place layers have overwritten
    // (device-to-device, on the stream).  Needs keep_inputs.
    int restoreInputs();

    size_t launchesPerStep() const { return ops.size() + 1; }
    // Algorithmic bytes of the GroupNorm, LayerNorm and GEGLU launches of one step.
    size_t bytesPerStep() const { return algorithmic_bytes; }

    // ---- what each launch works on, for checking a step against a reference implementation
    struct OpInfo {
        int kind;          // 0 GroupNorm+SiLU, 1 LayerNorm, 2 GEGLU, 3 SiLU
        size_t dims[2];    // GroupNorm {channels, hw}; LayerNorm {rows, dim}; GEGLU {rows, inner}; SiLU {n, 0}
        bool in_place;
    };
    size_t numOps() const { return ops.size(); }
    OpInfo opInfo(size_t i) const;
    std::vector<float> downloadInput(size_t i) const;
    std::vector<float> downloadOutput(size_t i) const;
    std::vector<float> downloadEmbedding() const;  // [batch, 320] of the last step
    // gamma and beta of launch i (empty for GEGLU / SiLU)
    const std::vector<float> &weight(size_t i) const { return ops.at(i).gamma; }
    const std::vector<float> &bias(size_t i) const { return ops.at(i).beta; }

private:
    struct Op {
        int kind;  // 0 GroupNorm+SiLU, 1 LayerNorm, 2 GEGLU, 3 SiLU
        size_t layer;
        size_t in, out;  // indices into buffers
        size_t dims[2];
        std::vector<float> gamma, beta;  // host copies of the synthetic affine
        size_t kept;                      // index into kept_inputs, or npos
    };
    static constexpr size_t npos = (size_t)-1;
    std::vector<DeviceBuffer> kept_inputs;
    bool keep_inputs;
    hipStream_t stream;
    size_t batch;
    DType dtype;
    std::vector<std::unique_ptr<GroupNorm>> group_norms;
    std::vector<std::unique_ptr<LayerNorm>> layer_norms;
    std::vector<std::unique_ptr<GEGLU>> geglus;
    std::vector<DeviceBuffer> buffers;
    std::vector<Op> ops;
    DeviceBuffer timestep_dev, embedding;
    size_t algorithmic_bytes = 0;
    hipGraph_t graph = nullptr;
    hipGraphExec_t graph_exec = nullptr;
};

}  // namespace msd
