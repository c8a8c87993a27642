// LayerNorm layer object: the drop-in for the reference's class LayerNorm
// (M/nn/LayerNorm.h:16-42).  Same construct / init() / forward() shape as GroupNorm.h;
// `eps` is an extension (the reference's kernel hard-codes 1e-5, K/layer_norm.cl:58).
#pragma once

#include <hip/hip_runtime_api.h>

#include <string>
#include <vector>

#include "DeviceBuffer.h"
#include "util.h"

namespace msd {

class LayerNorm {
public:
    LayerNorm(hipStream_t stream, size_t dim, const std::string &weight_name,
              const std::string &bias_name, float eps = 1e-5f);
    ~LayerNorm();
    LayerNorm(const LayerNorm &) = delete;
    LayerNorm &operator=(const LayerNorm &) = delete;

    // Throws std::runtime_error("weightSize != biasSize") / ("weightSize != weight->num_vals") /
    // ("weightSize % WORK_GROUP_SIZE != 0") like M/nn/LayerNorm.cpp:45-64.
    void init();
    void init(const std::vector<float> &weight, const std::vector<float> &bias);

    // input / output: [rows, dim], rows = elements / dim (M/nn/LayerNorm.cpp:73-85); throws
    // std::runtime_error("input_size % weight->num_vals != 0").  Returns 0 or a hipError_t.
    int forward(const DeviceBuffer &input, DeviceBuffer &output, unsigned num_events_in_list = 0,
                const hipEvent_t *event_wait_list = nullptr, hipEvent_t event = nullptr);
    // sum = a + b, output = LayerNorm(sum) in one launch: the elemwise_add the reference runs
    // before LayerNorm 2 and 3 (M/nn/BasicTransformerBlock.cpp:126-136,149-158) folded in; `sum`
    // is written because the block keeps it as its next residual, and may be `a` itself.
    // Equals elemwise_add followed by forward() bit for bit.
    int forwardAdd(const DeviceBuffer &a, const DeviceBuffer &b, DeviceBuffer &sum, DeviceBuffer &output,
                   unsigned num_events_in_list = 0, const hipEvent_t *event_wait_list = nullptr,
                   hipEvent_t event = nullptr);
    void checkInput(size_t input_bytes, DType dtype) const;

private:
    void logTiming(util::LaunchTimer &timer, size_t input_size, const char *kernel);
    DeviceBuffer bufferWeight;
    DeviceBuffer bufferBias;
    size_t weightSize;
    size_t biasSize;
    float eps;
    hipStream_t stream;
    const std::string weight_name;
    const std::string bias_name;
};

}  // namespace msd
