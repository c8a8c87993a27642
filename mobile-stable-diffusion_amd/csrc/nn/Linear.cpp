#include "Linear.h"

#include <hip/hip_runtime.h>

#include <stdexcept>

#include "util.h"

namespace msd {

Linear::Linear(hipStream_t stream, size_t in_features, size_t out_features, const std::string &weight_name,
               const std::string &bias_name, DType dtype)
    : weightShape({out_features, in_features}), dtype(dtype), stream(stream), weight_name(weight_name),
      bias_name(bias_name) {}

Linear::~Linear() = default;

void Linear::init() {
    if (!bufferWeight.empty() && (bias_name.empty() || !bufferBias.empty())) return;
    const npy::Array weight = util::load_npy_file(weight_name);
    std::vector<float> bias;
    if (!bias_name.empty()) bias = util::load_npy_file(bias_name).data;
    init(weight.data, bias);
}

void Linear::init(const std::vector<float> &weight, const std::vector<float> &bias) {
    if (!bufferWeight.empty()) return;
    if (weight.size() != weightShape[0] * weightShape[1])
        throw std::runtime_error("weight.num_vals != (weightShape[0] * weightShape[1])");
    if (!bias.empty() && bias.size() != weightShape[0])
        throw std::runtime_error("bias.num_vals != weightShape[0]");
    bufferWeight = util::upload(weight, dtype, stream);
    if (!bias.empty()) bufferBias = util::upload(bias, DType::F32, stream);
}

int Linear::forward(const DeviceBuffer &input, DeviceBuffer &output, unsigned num_events_in_list,
                    const hipEvent_t *event_wait_list, hipEvent_t event) {
    return forwardSilu(input, output, false, false, num_events_in_list, event_wait_list, event);
}

int Linear::forwardSilu(const DeviceBuffer &input, DeviceBuffer &output, bool silu_on_input,
                        bool silu_on_output, unsigned num_events_in_list,
                        const hipEvent_t *event_wait_list, hipEvent_t event) {
    if (bufferWeight.empty()) throw std::runtime_error("Linear: init() not called");
    if (input.ptr() == output.ptr()) throw std::runtime_error("Linear not support input == output");
    if (input.dtype() != dtype || output.dtype() != dtype)
        throw std::runtime_error("Linear: buffer storage type != weight storage type");
    const size_t inputSize = input.count();
    if (weightShape[1] == 0 || inputSize % weightShape[1] != 0)
        throw std::runtime_error("inputSize % weightShape[1] != 0");
    const size_t M = inputSize / weightShape[1], N = weightShape[0], K = weightShape[1];
    if (M > 8) throw std::runtime_error("Linear: more than 8 input rows is a GEMM, which this library leaves out");
    if (output.count() != M * N) throw std::runtime_error("Linear: output size != M * weightShape[0]");
    for (unsigned i = 0; i < num_events_in_list; i++) {
        const hipError_t err = hipStreamWaitEvent(stream, event_wait_list[i], 0);
        if (err != hipSuccess) return (int)err;
    }
    const int rc = msd_linear_rows(input.ptr(), bufferWeight.ptr(),
                                   bufferBias.empty() ? nullptr : static_cast<const float *>(bufferBias.ptr()),
                                   output.ptr(), M, N, K, silu_on_input ? MSD_ACT_SILU : MSD_ACT_NONE,
                                   silu_on_output ? MSD_ACT_SILU : MSD_ACT_NONE, (int)dtype, stream);
    if (rc != MSD_OK) return rc;
    if (event) return (int)hipEventRecord(event, stream);
    return MSD_OK;
}

int Linear::forwardSiluGrouped(const std::vector<Linear *> &layers, const DeviceBuffer &input,
                               std::vector<DeviceBuffer> &outputs, bool silu_on_input, bool silu_on_output,
                               unsigned num_events_in_list, const hipEvent_t *event_wait_list,
                               hipEvent_t event) {
    if (layers.empty()) return MSD_OK;
    if (layers.size() != outputs.size()) throw std::runtime_error("Linear: one output per layer");
    const Linear &first = *layers[0];
    const size_t K = first.weightShape[1];
    if (K == 0 || input.count() % K != 0) throw std::runtime_error("inputSize % weightShape[1] != 0");
    const size_t M = input.count() / K;
    if (M > 8) throw std::runtime_error("Linear: more than 8 input rows is a GEMM, which this library leaves out");
    std::vector<const void *> ws(layers.size());
    std::vector<const float *> bs(layers.size());
    std::vector<void *> ys(layers.size());
    std::vector<size_t> ns(layers.size());
    for (size_t i = 0; i < layers.size(); i++) {
        const Linear &l = *layers[i];
        if (l.bufferWeight.empty()) throw std::runtime_error("Linear: init() not called");
        if (l.weightShape[1] != K || l.dtype != first.dtype || l.stream != first.stream)
            throw std::runtime_error("Linear: grouped layers differ in in_features, storage type or stream");
        if (input.dtype() != l.dtype || outputs[i].dtype() != l.dtype)
            throw std::runtime_error("Linear: buffer storage type != weight storage type");
        if (input.ptr() == outputs[i].ptr()) throw std::runtime_error("Linear not support input == output");
        if (outputs[i].count() != M * l.weightShape[0])
            throw std::runtime_error("Linear: output size != M * weightShape[0]");
        ws[i] = l.bufferWeight.ptr();
        bs[i] = l.bufferBias.empty() ? nullptr : static_cast<const float *>(l.bufferBias.ptr());
        ys[i] = outputs[i].ptr();
        ns[i] = l.weightShape[0];
    }
    for (unsigned i = 0; i < num_events_in_list; i++) {
        const hipError_t err = hipStreamWaitEvent(first.stream, event_wait_list[i], 0);
        if (err != hipSuccess) return (int)err;
    }
    const int rc = msd_linear_rows_grouped(input.ptr(), ws.data(), bs.data(), ys.data(), ns.data(), layers.size(), M,
                                           K, silu_on_input ? MSD_ACT_SILU : MSD_ACT_NONE,
                                           silu_on_output ? MSD_ACT_SILU : MSD_ACT_NONE, (int)first.dtype,
                                           first.stream);
    if (rc != MSD_OK) return rc;
    if (event) return (int)hipEventRecord(event, first.stream);
    return MSD_OK;
}

}  // namespace msd
