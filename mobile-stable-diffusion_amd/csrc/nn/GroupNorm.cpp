#include "GroupNorm.h"

#include <hip/hip_runtime.h>

#include <cstdio>
#include <stdexcept>
#include <string>

#include "util.h"

#define WORK_GROUP_SIZE 64  // the reference's reduction width (M/nn/GroupNorm.cpp:13)

namespace msd {

GroupNorm::GroupNorm(hipStream_t stream, size_t num_groups, size_t num_channels, float eps,
                     const std::string &weight_name, const std::string &bias_name, size_t batch,
                     bool fuse_silu)
    : weightSize(num_channels), biasSize(num_channels), num_groups(num_groups),
      num_channels(num_channels), eps(eps), batch(batch), fuse_silu(fuse_silu), stream(stream),
      weight_name(weight_name), bias_name(bias_name) {}

GroupNorm::~GroupNorm() = default;  // the buffers free their memory

void GroupNorm::init() {
    if (!bufferWeight.empty() && !bufferBias.empty()) return;
    const npy::Array weight = util::load_npy_file(weight_name);
    const npy::Array bias = util::load_npy_file(bias_name);
    init(weight.data, bias.data);
}

void GroupNorm::init(const std::vector<float> &weight, const std::vector<float> &bias) {
    if (!bufferWeight.empty() && !bufferBias.empty()) return;
    if (weight.size() != bias.size()) throw std::runtime_error("weight.shape[0] != bias.shape[0]");
    if (weight.size() != weightSize) throw std::runtime_error("weight.shape[0] != weightSize");
    bufferWeight = util::upload(weight, DType::F32, stream);
    bufferBias = util::upload(bias, DType::F32, stream);
    const int rc = msd_init(stream);  // scratch now, so forward() never allocates
    if (rc != MSD_OK) throw std::runtime_error(std::string("msd_init: ") + msd_error_string(rc));
}

void GroupNorm::checkInput(size_t input_bytes, DType dtype) const {
    if (batch == 0 || num_groups == 0) throw std::runtime_error("batch and num_groups must be positive");
    const size_t total = input_bytes / dtype_size(dtype);
    if (total % batch != 0) throw std::runtime_error("input_size % batch != 0");
    const size_t input_size = total / batch;  // one sample: what the reference calls input_size
    const size_t groupSize = input_size / num_groups;
    if (input_size % weightSize != 0) throw std::runtime_error("input_size % weight->num_vals != 0");
    if (groupSize % WORK_GROUP_SIZE != 0) throw std::runtime_error("groupSize % WORK_GROUP_SIZE != 0");
    if (weightSize % num_groups != 0) throw std::runtime_error("num_channels % num_groups != 0");
}

int GroupNorm::forward(const DeviceBuffer &input, DeviceBuffer &output, unsigned num_events_in_list,
                       const hipEvent_t *event_wait_list, hipEvent_t event) {
    return run(input, nullptr, output, num_events_in_list, event_wait_list, event);
}

int GroupNorm::forward(const DeviceBuffer &input, const DeviceBuffer &chunk, DeviceBuffer &output,
                       unsigned num_events_in_list, const hipEvent_t *event_wait_list,
                       hipEvent_t event) {
    if (chunk.dtype() != input.dtype() || chunk.count() != batch * num_channels)
        throw std::runtime_error("chunk size != batch * num_channels");
    return run(input, &chunk, output, num_events_in_list, event_wait_list, event);
}

int GroupNorm::forwardTokens(const DeviceBuffer &input, DeviceBuffer &output, unsigned num_events_in_list,
                             const hipEvent_t *event_wait_list, hipEvent_t event) {
    if (bufferWeight.empty() || bufferBias.empty()) throw std::runtime_error("GroupNorm: init() not called");
    checkInput(input.bytes(), input.dtype());
    if (output.bytes() != input.bytes() || output.dtype() != input.dtype() || output.ptr() == input.ptr())
        throw std::runtime_error("output must be separate memory of the input's size / type");
    for (unsigned i = 0; i < num_events_in_list; i++) {
        const hipError_t err = hipStreamWaitEvent(stream, event_wait_list[i], 0);
        if (err != hipSuccess) return (int)err;
    }
    const size_t channelSize = input.count() / batch / num_channels;
    const int rc = msd_groupnorm_tokens(input.ptr(), output.ptr(), static_cast<const float *>(bufferWeight.ptr()),
                                        static_cast<const float *>(bufferBias.ptr()), batch, num_channels,
                                        channelSize, num_groups, eps, (int)input.dtype(), stream);
    if (rc != MSD_OK) return rc;
    if (event) return (int)hipEventRecord(event, stream);
    return MSD_OK;
}

int GroupNorm::run(const DeviceBuffer &input, const DeviceBuffer *chunk, DeviceBuffer &output,
                   unsigned num_events_in_list, const hipEvent_t *event_wait_list, hipEvent_t event) {
    if (bufferWeight.empty() || bufferBias.empty()) throw std::runtime_error("GroupNorm: init() not called");
    checkInput(input.bytes(), input.dtype());
    if (output.bytes() != input.bytes() || output.dtype() != input.dtype())
        throw std::runtime_error("output size / type != input size / type");
    for (unsigned i = 0; i < num_events_in_list; i++) {
        const hipError_t err = hipStreamWaitEvent(stream, event_wait_list[i], 0);
        if (err != hipSuccess) return (int)err;
    }
    const size_t input_size = input.count() / batch;
    const size_t channelSize = input_size / num_channels;  // H*W (M/nn/GroupNorm.cpp:130)
    const float *w = static_cast<const float *>(bufferWeight.ptr());
    const float *b = static_cast<const float *>(bufferBias.ptr());
    util::LaunchTimer timer(stream);
    const int rc = chunk ? msd_chunk_add_groupnorm(input.ptr(), chunk->ptr(), output.ptr(), w, b, batch,
                                                   num_channels, channelSize, num_groups, eps,
                                                   fuse_silu ? 1 : 0, (int)input.dtype(), stream)
                         : msd_groupnorm(input.ptr(), output.ptr(), w, b, batch, num_channels,
                                         channelSize, num_groups, eps, fuse_silu ? 1 : 0,
                                         (int)input.dtype(), stream);
    if (rc != MSD_OK) return rc;
    if (util::debugTiming()) {
        // the reference's row (M/nn/GroupNorm.cpp:149-161), one kernel instead of three
        static int count = 0;
        if (count == 0)
            fprintf(stderr, "try, component, index, input size, group size, num group, weight size, "
                            "workgroup size, kernel, time(ms)\n");
        const std::string message = "0, GroupNorm, " + std::to_string(count++) + ", " +
                                    std::to_string(input_size) + ", " +
                                    std::to_string(input_size / num_groups) + ", " +
                                    std::to_string(num_groups) + ", " + std::to_string(weightSize) + ", " +
                                    std::to_string(WORK_GROUP_SIZE);
        timer.finish(message + (chunk ? ", chunk_add_group_norm" : ", group_norm") +
                     (fuse_silu ? "_silu" : ""));
    }
    if (event) return (int)hipEventRecord(event, stream);
    return MSD_OK;
}

}  // namespace msd
