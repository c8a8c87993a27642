#include "LayerNorm.h"

#include <hip/hip_runtime.h>

#include <stdexcept>
#include <string>

#include "util.h"

#define WORK_GROUP_SIZE 64  // M/nn/LayerNorm.cpp:11

namespace msd {

LayerNorm::LayerNorm(hipStream_t stream, size_t dim, const std::string &weight_name,
                     const std::string &bias_name, float eps)
    : weightSize(dim), biasSize(dim), eps(eps), stream(stream), weight_name(weight_name),
      bias_name(bias_name) {}

LayerNorm::~LayerNorm() = default;

void LayerNorm::init() {
    if (!bufferWeight.empty() && !bufferBias.empty()) return;
    const npy::Array weight = util::load_npy_file(weight_name);
    const npy::Array bias = util::load_npy_file(bias_name);
    init(weight.data, bias.data);
}

void LayerNorm::init(const std::vector<float> &weight, const std::vector<float> &bias) {
    if (!bufferWeight.empty() && !bufferBias.empty()) return;
    if (weight.size() != bias.size()) throw std::runtime_error("weightSize != biasSize");
    if (weight.size() != weightSize) throw std::runtime_error("weightSize != weight->num_vals");
    if (weightSize % WORK_GROUP_SIZE != 0) throw std::runtime_error("weightSize % WORK_GROUP_SIZE != 0");
    bufferWeight = util::upload(weight, DType::F32, stream);
    bufferBias = util::upload(bias, DType::F32, stream);
}

// The reference's timing row (M/nn/LayerNorm.cpp:144-154), one kernel instead of three.
void LayerNorm::logTiming(util::LaunchTimer &timer, size_t input_size, const char *kernel) {
    if (!util::debugTiming()) return;
    static int count = 0;
    timer.finish("2, LayerNorm, " + std::to_string(count++) + ", " + std::to_string(input_size) + ", " +
                 std::to_string(weightSize) + ", " + kernel);
}

void LayerNorm::checkInput(size_t input_bytes, DType dtype) const {
    const size_t input_size = input_bytes / dtype_size(dtype);
    if (weightSize == 0 || input_size % weightSize != 0)
        throw std::runtime_error("input_size % weight->num_vals != 0");
}

int LayerNorm::forward(const DeviceBuffer &input, DeviceBuffer &output, unsigned num_events_in_list,
                       const hipEvent_t *event_wait_list, hipEvent_t event) {
    if (bufferWeight.empty() || bufferBias.empty()) throw std::runtime_error("LayerNorm: init() not called");
    checkInput(input.bytes(), input.dtype());
    if (output.bytes() != input.bytes() || output.dtype() != input.dtype())
        throw std::runtime_error("output size / type != input size / type");
    for (unsigned i = 0; i < num_events_in_list; i++) {
        const hipError_t err = hipStreamWaitEvent(stream, event_wait_list[i], 0);
        if (err != hipSuccess) return (int)err;
    }
    util::LaunchTimer timer(stream);
    const int rc = msd_layernorm(input.ptr(), output.ptr(), static_cast<const float *>(bufferWeight.ptr()),
                                 static_cast<const float *>(bufferBias.ptr()), input.count() / weightSize,
                                 weightSize, eps, (int)input.dtype(), stream);
    if (rc != MSD_OK) return rc;
    logTiming(timer, input.count(), "layer_norm");
    if (event) return (int)hipEventRecord(event, stream);
    return MSD_OK;
}

int LayerNorm::forwardAdd(const DeviceBuffer &a, const DeviceBuffer &b, DeviceBuffer &sum,
                          DeviceBuffer &output, unsigned num_events_in_list,
                          const hipEvent_t *event_wait_list, hipEvent_t event) {
    if (bufferWeight.empty() || bufferBias.empty()) throw std::runtime_error("LayerNorm: init() not called");
    checkInput(a.bytes(), a.dtype());
    if (b.bytes() != a.bytes() || sum.bytes() != a.bytes() || output.bytes() != a.bytes() ||
        b.dtype() != a.dtype() || sum.dtype() != a.dtype() || output.dtype() != a.dtype())
        throw std::runtime_error("operand sizes / types differ");
    for (unsigned i = 0; i < num_events_in_list; i++) {
        const hipError_t err = hipStreamWaitEvent(stream, event_wait_list[i], 0);
        if (err != hipSuccess) return (int)err;
    }
    util::LaunchTimer timer(stream);
    const int rc = msd_add_layernorm(a.ptr(), b.ptr(), sum.ptr(), output.ptr(),
                                     static_cast<const float *>(bufferWeight.ptr()),
                                     static_cast<const float *>(bufferBias.ptr()), a.count() / weightSize,
                                     weightSize, eps, (int)a.dtype(), stream);
    if (rc != MSD_OK) return rc;
    logTiming(timer, a.count(), "add_layer_norm");
    if (event) return (int)hipEventRecord(event, stream);
    return MSD_OK;
}

}  // namespace msd
