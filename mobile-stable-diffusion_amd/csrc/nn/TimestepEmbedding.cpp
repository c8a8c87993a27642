#include "TimestepEmbedding.h"

#include <hip/hip_runtime.h>

#include <cstdint>
#include <stdexcept>

namespace msd {

DeviceBuffer createTimestepEmbedding(hipStream_t stream, const std::vector<long> &timesteps,
                                     DType dtype, int dim, float max_period) {
    const size_t batch = timesteps.size();
    DeviceBuffer out = DeviceBuffer::allocate(batch * (size_t)dim * dtype_size(dtype), dtype);
    if (batch == 0) return out;
    std::vector<int64_t> host(timesteps.begin(), timesteps.end());
    DeviceBuffer t = DeviceBuffer::allocate(batch * sizeof(int64_t), DType::F32);
    hipError_t err = hipMemcpyAsync(t.ptr(), host.data(), batch * sizeof(int64_t),
                                    hipMemcpyHostToDevice, stream);
    if (err != hipSuccess)
        throw std::runtime_error(std::string("createTimestepEmbedding: ") + hipGetErrorString(err));
    const int rc = msd_timestep_embedding(static_cast<const int64_t *>(t.ptr()), out.ptr(), batch,
                                          (size_t)dim, max_period, (int)dtype, stream);
    if (rc != MSD_OK)
        throw std::runtime_error(std::string("createTimestepEmbedding: ") + msd_error_string(rc));
    err = hipStreamSynchronize(stream);  // `host` and `t` go out of scope
    if (err != hipSuccess)
        throw std::runtime_error(std::string("createTimestepEmbedding: ") + hipGetErrorString(err));
    return out;
}

std::vector<int> ddimTimesteps(int ddim_num_steps) {
    const int n = msd_ddim_timesteps(ddim_num_steps, nullptr, 0);
    if (n < 0) throw std::runtime_error("ddim_num_steps must be in [1, 1000]");
    std::vector<int> out((size_t)n);
    msd_ddim_timesteps(ddim_num_steps, out.data(), n);
    return out;
}

}  // namespace msd
