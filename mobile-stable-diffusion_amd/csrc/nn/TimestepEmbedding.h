// Sinusoidal timestep embedding and the integer DDIM timestep list.
//   createTimestepEmbedding  UNetModel::createTimestepEmbedding (M/UNetModel.cpp:1935-1958):
//                            returns a fresh device buffer [batch, MODEL_CHANNELS] as the
//                            reference returns a fresh cl_mem; computed on the device.
//   ddimTimesteps            the list DDIMSampler::sample builds (M/DDIMSampler.cpp:60-64).
#pragma once

#include <hip/hip_runtime_api.h>

#include <vector>

#include "DeviceBuffer.h"

namespace msd {

constexpr int MODEL_CHANNELS = 320;  // M/UNetModel.cpp:12

// One timestep per sample (the reference takes a single `long` for its batch of one).
// Throws std::runtime_error on failure.
DeviceBuffer createTimestepEmbedding(hipStream_t stream, const std::vector<long> &timesteps,
                                     DType dtype = DType::F32, int dim = MODEL_CHANNELS,
                                     float max_period = 10000.0f);
inline DeviceBuffer createTimestepEmbedding(hipStream_t stream, long timestep) {
    return createTimestepEmbedding(stream, std::vector<long>{timestep});
}

// Ascending {1, 1+c, ...}, c = 1000 / ddim_num_steps; the sampler consumes it from the back.
// Throws std::runtime_error for steps outside [1, 1000].
std::vector<int> ddimTimesteps(int ddim_num_steps);

}  // namespace msd
