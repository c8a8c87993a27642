// GEGLU layer object: the gelu_multiply half of the reference's class GEGLU
// (M/nn/GEGLU.h:18-44, M/nn/GEGLU.cpp:47-84).  The reference's GEGLU owns the
// Linear(in_features, 2*out_features) that produces the projection; that GEMM is outside
// this library, so forward() takes the already projected tensor [rows, 2*out_features]
// (value | gate) and writes [rows, out_features].
#pragma once

#include <hip/hip_runtime_api.h>

#include <vector>

#include "DeviceBuffer.h"

namespace msd {

class GEGLU {
public:
    GEGLU(hipStream_t stream, size_t in_features, size_t out_features);

    void init() {}  // nothing to load: kept so call sites read like the reference's

    // projected: [rows, 2*out_features]; output: [rows, out_features]; rows = elements /
    // weightShape[0] as in M/nn/GEGLU.cpp:59,75.  Throws std::runtime_error when the sizes do
    // not divide.  Returns 0 or a hipError_t value.
    int forward(const DeviceBuffer &projected, DeviceBuffer &output, unsigned num_events_in_list = 0,
                const hipEvent_t *event_wait_list = nullptr, hipEvent_t event = nullptr);
    void checkInput(size_t projected_bytes, size_t output_bytes, DType dtype) const;

    // Shape of the projection weight the caller's Linear holds: {2*out_features, in_features}
    // (the reference exposes linear->weightShape the same way, M/nn/GEGLU.h:36).
    std::vector<size_t> weightShape;

private:
    hipStream_t stream;
};

}  // namespace msd
