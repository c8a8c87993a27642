// DDIM sampler: the drop-in for the reference's class DDIMSampler (M/DDIMSampler.h:10-41)
// with the latent kept on the device.  Same assumptions as the reference's p_sample_ddim
// (M/DDIMSampler.cpp:90-93): eta = 0, guidance scale 1, one conditioning.
#pragma once

#include <hip/hip_runtime_api.h>

#include <functional>
#include <utility>
#include <vector>

#include "DeviceBuffer.h"

namespace msd {

class DDIMSampler {
public:
    // apply_model(x, t, conditioning, e_t) writes the predicted noise for latent x at timestep
    // t into e_t (same size and type as x) on the sampler's stream and returns 0 or an error
    // code; it stands where the reference passes UNetModel::forward as a std::function
    // returning a host vector (M/DDIMSampler.cpp:18-20, 105).
    typedef std::function<int(const DeviceBuffer &x, int t, const DeviceBuffer &conditioning,
                              DeviceBuffer &e_t)> ApplyModel;

    DDIMSampler(hipStream_t stream, ApplyModel apply_model);
    ~DDIMSampler();

    // Runs ddim_num_steps updates from x_T (copied, float32 or float16) and returns the final
    // latent.  x_T == nullptr draws N(0, 1) noise of shape[0] * shape[1] * shape[2] from
    // std::mt19937(42) as M/DDIMSampler.cpp:49-56 does; that draw depends on the C++ library's
    // std::normal_distribution and is not reproducible across standard libraries.
    // Throws std::runtime_error for ddim_num_steps outside [1, 500] and for failures.
    DeviceBuffer sample(const DeviceBuffer *x_T, int ddim_num_steps, const int shape[3],
                        const DeviceBuffer &conditioning);

    // make_schedule (M/DDIMSampler.cpp:123-137): alphas, alphas_prev for a timestep list.
    std::pair<std::vector<float>, std::vector<float>> make_schedule(const std::vector<int> &ddim_timesteps) const;

    const std::vector<float> &alphasCumprod() const { return alphas_cumprod; }

private:
    // One update in place (M/DDIMSampler.cpp:94-121); e_t is scratch of the size of x.
    int p_sample_ddim(DeviceBuffer &x, int t, const DeviceBuffer &c, size_t index, const std::vector<float> &alphas,
                      const std::vector<float> &alphas_prev, const std::vector<float> &sqrt_one_minus_alphas,
                      DeviceBuffer &e_t);

    std::vector<float> alphas_cumprod;
    hipStream_t stream;
    const ApplyModel apply_model;
};

}  // namespace msd
