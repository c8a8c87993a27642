#include "GEGLU.h"

#include <hip/hip_runtime.h>

#include <stdexcept>

namespace msd {

GEGLU::GEGLU(hipStream_t stream, size_t in_features, size_t out_features)
    : weightShape{out_features * 2, in_features}, stream(stream) {}

void GEGLU::checkInput(size_t projected_bytes, size_t output_bytes, DType dtype) const {
    const size_t width = weightShape[0];
    const size_t n = projected_bytes / dtype_size(dtype);
    if (width == 0 || n % width != 0) throw std::runtime_error("input_size % (2 * out_features) != 0");
    if (output_bytes != projected_bytes / 2) throw std::runtime_error("output size != input size / 2");
}

int GEGLU::forward(const DeviceBuffer &projected, DeviceBuffer &output, unsigned num_events_in_list,
                   const hipEvent_t *event_wait_list, hipEvent_t event) {
    checkInput(projected.bytes(), output.bytes(), projected.dtype());
    if (output.dtype() != projected.dtype()) throw std::runtime_error("output type != input type");
    {   // the kernel reads proj rows and writes out rows of another stride: they must not overlap
        const char *p0 = static_cast<const char *>(projected.ptr());
        const char *o0 = static_cast<const char *>(output.ptr());
        if (projected.bytes() != 0 && o0 < p0 + projected.bytes() && p0 < o0 + output.bytes())
            throw std::runtime_error("GEGLU not support input overlapping output");
    }
    for (unsigned i = 0; i < num_events_in_list; i++) {
        const hipError_t err = hipStreamWaitEvent(stream, event_wait_list[i], 0);
        if (err != hipSuccess) return (int)err;
    }
    const size_t rows = projected.count() / weightShape[0];  // M/nn/GEGLU.cpp:75
    const int rc = msd_geglu(projected.ptr(), output.ptr(), rows, weightShape[0] / 2,
                             (int)projected.dtype(), stream);
    if (rc != MSD_OK) return rc;
    if (event) return (int)hipEventRecord(event, stream);
    return MSD_OK;
}

}  // namespace msd
