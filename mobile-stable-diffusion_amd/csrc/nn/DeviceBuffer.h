// A device allocation that carries its byte size and storage type, standing in for the
// reference's cl_mem: its layers derive every shape from the buffer size
// (clGetMemObjectInfo(CL_MEM_SIZE), M/nn/GroupNorm.cpp:76-81, M/nn/LayerNorm.cpp:73-76,
// M/nn/GEGLU.cpp:56-59), so the handle has to know it.
#pragma once

#include <cstddef>
#include <stdexcept>

#include "msd_hip.h"

namespace msd {

enum class DType : int { F32 = MSD_DTYPE_F32, F16 = MSD_DTYPE_F16 };

inline size_t dtype_size(DType t) { return t == DType::F16 ? 2 : 4; }

class DeviceBuffer {
public:
    DeviceBuffer() = default;
    // Wraps memory the caller owns (nothing is freed).
    DeviceBuffer(void *ptr, size_t bytes, DType dtype) : ptr_(ptr), bytes_(bytes), dtype_(dtype) {}
    // Allocates `bytes` of device memory owned by the buffer; throws std::runtime_error.
    static DeviceBuffer allocate(size_t bytes, DType dtype);

    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    DeviceBuffer(DeviceBuffer &&o) noexcept { *this = static_cast<DeviceBuffer &&>(o); }
    DeviceBuffer &operator=(DeviceBuffer &&o) noexcept;
    ~DeviceBuffer();

    void *ptr() const { return ptr_; }
    size_t bytes() const { return bytes_; }
    DType dtype() const { return dtype_; }
    size_t count() const { return bytes_ / dtype_size(dtype_); }  // elements
    bool empty() const { return ptr_ == nullptr; }
    void release();

private:
    void *ptr_ = nullptr;
    size_t bytes_ = 0;
    DType dtype_ = DType::F32;
    bool owned_ = false;
};

}  // namespace msd
