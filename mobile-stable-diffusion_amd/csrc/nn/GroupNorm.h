// GroupNorm layer object: the drop-in for the reference's class GroupNorm
// (M/nn/GroupNorm.h:15-47): construct with the weight file names, init() loads them,
// forward(input, output) enqueues the work.  cl_context + cl_command_queue become a
// hipStream_t, cl_mem becomes DeviceBuffer, the shared GroupNormKernel holder disappears
// (the kernels are linked in).  Extensions the reference lacks: `batch` (its forward
// assumes one sample, M/nn/GroupNorm.cpp:79-80), `fuse_silu` (it runs SiLU as a separate
// kernel, M/nn/ResBlock.cpp:136-142) and fp16 storage.
#pragma once

#include <hip/hip_runtime_api.h>

#include <string>
#include <vector>

#include "DeviceBuffer.h"

namespace msd {

class GroupNorm {
public:
    GroupNorm(hipStream_t stream, size_t num_groups, size_t num_channels, float eps,
              const std::string &weight_name, const std::string &bias_name, size_t batch = 1,
              bool fuse_silu = false);
    ~GroupNorm();
    GroupNorm(const GroupNorm &) = delete;
    GroupNorm &operator=(const GroupNorm &) = delete;

    // Loads weight and bias (float32 .npy, [num_channels]) once; later calls return at once
    // (M/nn/GroupNorm.cpp:51-66).  Throws std::runtime_error("weight.shape[0] != bias.shape[0]")
    // / ("weight.shape[0] != weightSize") like the reference, or the loader's error.
    void init();
    // Same, from host arrays (no reference counterpart; for synthetic weights).
    void init(const std::vector<float> &weight, const std::vector<float> &bias);

    // input / output: [batch, num_channels, H*W] in the buffers' storage type; output may be
    // the same memory as input.  Shapes come from the buffer size as in the reference.  The
    // work runs on the stream after the events in event_wait_list; `event`, when not null, is
    // recorded behind it.  Returns 0 or a hipError_t value; throws std::runtime_error on the
    // reference's preconditions ("input_size % weight->num_vals != 0",
    // "groupSize % WORK_GROUP_SIZE != 0", M/nn/GroupNorm.cpp:83-93).
    int forward(const DeviceBuffer &input, DeviceBuffer &output, unsigned num_events_in_list = 0,
                const hipEvent_t *event_wait_list = nullptr, hipEvent_t event = nullptr);

    // forward() on input + chunk, chunk = one value per (sample, channel) broadcast over H*W:
    // the chunkwise_add the reference's ResBlock runs right before its out-norm
    // (M/nn/ResBlock.cpp:188-199, then :222) folded into the same launch.  The result equals
    // chunkwise_add followed by forward() bit for bit.  chunk holds batch * num_channels
    // elements of the input's storage type.
    int forward(const DeviceBuffer &input, const DeviceBuffer &chunk, DeviceBuffer &output,
                unsigned num_events_in_list = 0, const hipEvent_t *event_wait_list = nullptr,
                hipEvent_t event = nullptr);

    // GroupNorm stored token-major: output[b, p, c] = GroupNorm(input)[b, c, p], i.e. forward()
    // followed by the (0, 2, 1) permute of SpatialTransformer::forward
    // (M/nn/SpatialTransformer.cpp:127-139) in one launch.  Never applies SiLU.  output must
    // be different memory of the same size.
    int forwardTokens(const DeviceBuffer &input, DeviceBuffer &output, unsigned num_events_in_list = 0,
                      const hipEvent_t *event_wait_list = nullptr, hipEvent_t event = nullptr);

    // The precondition checks of forward() alone (no device work).
    void checkInput(size_t input_bytes, DType dtype) const;

private:
    int run(const DeviceBuffer &input, const DeviceBuffer *chunk, DeviceBuffer &output,
            unsigned num_events_in_list, const hipEvent_t *event_wait_list, hipEvent_t event);
    DeviceBuffer bufferWeight;
    DeviceBuffer bufferBias;
    size_t weightSize;
    size_t biasSize;
    size_t num_groups;
    size_t num_channels;
    float eps;
    size_t batch;
    bool fuse_silu;
    hipStream_t stream;
    const std::string weight_name;
    const std::string bias_name;
};

}  // namespace msd
