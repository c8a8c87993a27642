// Linear layer object for the rows of the time embedding: the drop-in for the reference's
// class Linear (M/nn/Linear.h:18-50) at its embedding call sites: time_embed_0 / time_embed_2
// (M/UNetModel.cpp:1107-1120) and each ResBlock's embed_linear (M/nn/ResBlock.cpp:173-183).
// Same construct / init() / forward() shape; the context and the shared kernel holders are
// gone.  Inputs of more than 8 rows are GEMMs and are refused.
#pragma once

#include <hip/hip_runtime_api.h>

#include <string>
#include <vector>

#include "DeviceBuffer.h"

namespace msd {

class Linear {
public:
    // `dtype` is the storage type of the weight on the device; inputs and outputs of forward()
    // must use the same one.  The bias (bias_name may be empty, as in the reference) stays float32.
    Linear(hipStream_t stream, size_t in_features, size_t out_features, const std::string &weight_name,
           const std::string &bias_name, DType dtype = DType::F32);
    ~Linear();
    Linear(const Linear &) = delete;
    Linear &operator=(const Linear &) = delete;

    // Loads the .npy files.  Throws std::runtime_error("weight.num_vals != (weightShape[0] *
    // weightShape[1])") / ("bias.num_vals != weightShape[0]") like M/nn/Linear.cpp:48-71.
    void init();
    void init(const std::vector<float> &weight, const std::vector<float> &bias);

    // output[M, N] = input[M, K] . weight[N, K]^T + bias, M = elements / K (M/nn/Linear.cpp:83-97).
    // Throws std::runtime_error("Linear not support input == output") and
    // ("inputSize % weightShape[1] != 0") as the reference does, and for M > 8.
    int forward(const DeviceBuffer &input, DeviceBuffer &output, unsigned num_events_in_list = 0,
                const hipEvent_t *event_wait_list = nullptr, hipEvent_t event = nullptr);
    // The same with the silu enqueue that the embedding call sites place before
    // (M/nn/ResBlock.cpp:173-180) or behind (M/UNetModel.cpp:1110-1117) the layer folded in.
    int forwardSilu(const DeviceBuffer &input, DeviceBuffer &output, bool silu_on_input,
                    bool silu_on_output, unsigned num_events_in_list = 0,
                    const hipEvent_t *event_wait_list = nullptr, hipEvent_t event = nullptr);

    // Several layers on the SAME input rows in one launch: outputs[i] = layers[i](input), each
    // exactly what its own forwardSilu() call gives.  For the embed_linear of all ResBlocks of a
    // UNet step, which the reference runs one by one on the same emb (M/nn/ResBlock.cpp:173-183;
    // emb exists once M/UNetModel.cpp:1107-1120 has run): call it once ahead of the blocks.
    // All layers share in_features, the storage type and the stream; throws what forwardSilu throws.
    static int forwardSiluGrouped(const std::vector<Linear *> &layers, const DeviceBuffer &input,
                                  std::vector<DeviceBuffer> &outputs, bool silu_on_input, bool silu_on_output,
                                  unsigned num_events_in_list = 0, const hipEvent_t *event_wait_list = nullptr,
                                  hipEvent_t event = nullptr);

    std::vector<size_t> weightShape;  // {out_features, in_features}

private:
    DeviceBuffer bufferWeight;
    DeviceBuffer bufferBias;  // empty when the layer has no bias
    DType dtype;
    hipStream_t stream;
    const std::string weight_name;
    const std::string bias_name;
};

}  // namespace msd
