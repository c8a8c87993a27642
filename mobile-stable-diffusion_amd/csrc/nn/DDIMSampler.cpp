#include "DDIMSampler.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <random>
#include <stdexcept>
#include <string>

#include "TimestepEmbedding.h"
#include "util.h"

#define DDPM_NUM_TIME_STEPS 1000  // M/DDIMSampler.cpp:13
#define SEED 42                   // M/DDIMSampler.cpp:14

namespace msd {

DDIMSampler::DDIMSampler(hipStream_t stream, ApplyModel apply_model)
    : alphas_cumprod(DDPM_NUM_TIME_STEPS), stream(stream), apply_model(std::move(apply_model)) {
    if (msd_alphas_cumprod(alphas_cumprod.data()) != MSD_OK) throw std::runtime_error("alphas_cumprod failed");
}

DDIMSampler::~DDIMSampler() = default;

std::pair<std::vector<float>, std::vector<float>> DDIMSampler::make_schedule(
    const std::vector<int> &ddim_timesteps) const {
    std::vector<float> alphas, alphas_prev;
    for (size_t i = 0; i < ddim_timesteps.size(); i++) {
        const int step = ddim_timesteps[i];
        if (step < 0 || step >= DDPM_NUM_TIME_STEPS) throw std::runtime_error("timestep outside the alpha table");
        alphas.push_back(alphas_cumprod[(size_t)step]);
        alphas_prev.push_back(i == 0 ? alphas_cumprod[0] : alphas_cumprod[(size_t)ddim_timesteps[i - 1]]);
    }
    return std::make_pair(alphas, alphas_prev);
}

DeviceBuffer DDIMSampler::sample(const DeviceBuffer *x_T, int ddim_num_steps, const int shape[3],
                                 const DeviceBuffer &conditioning) {
    if (ddim_num_steps < 1 || ddim_num_steps > DDPM_NUM_TIME_STEPS / 2)
        throw std::runtime_error("ddim_num_steps must be in [1, 500]");
    DeviceBuffer img;
    if (x_T == nullptr) {
        std::mt19937 gen(SEED);
        std::normal_distribution<float> normalDist(0.0f, 1.0f);
        std::vector<float> host((size_t)shape[0] * shape[1] * shape[2]);
        for (float &v : host) v = normalDist(gen);
        img = util::upload(host, DType::F32, stream);
    } else {
        img = DeviceBuffer::allocate(x_T->bytes(), x_T->dtype());
        const hipError_t err = hipMemcpyAsync(img.ptr(), x_T->ptr(), x_T->bytes(), hipMemcpyDeviceToDevice, stream);
        if (err != hipSuccess) throw std::runtime_error(std::string("sample: ") + hipGetErrorString(err));
    }
    DeviceBuffer e_t = DeviceBuffer::allocate(img.bytes(), img.dtype());

    const std::vector<int> ddim_timesteps = ddimTimesteps(ddim_num_steps);
    const auto schedule = make_schedule(ddim_timesteps);
    const std::vector<float> &alphas = schedule.first;
    const std::vector<float> &alphas_prev = schedule.second;
    std::vector<float> sqrt_one_minus_alphas(alphas.size());
    for (size_t i = 0; i < alphas.size(); i++) sqrt_one_minus_alphas[i] = std::sqrt(1.0f - alphas[i]);

    for (int index = static_cast<int>(ddim_timesteps.size()) - 1; index >= 0; index--) {
        const int rc = p_sample_ddim(img, ddim_timesteps[(size_t)index], conditioning, (size_t)index, alphas,
                                     alphas_prev, sqrt_one_minus_alphas, e_t);
        if (rc != MSD_OK) throw std::runtime_error(std::string("p_sample_ddim: ") + msd_error_string(rc));
    }
    const hipError_t err = hipStreamSynchronize(stream);  // e_t is released on return
    if (err != hipSuccess) throw std::runtime_error(std::string("sample: ") + hipGetErrorString(err));
    return img;
}

int DDIMSampler::p_sample_ddim(DeviceBuffer &x, int t, const DeviceBuffer &c, size_t index,
                               const std::vector<float> &alphas, const std::vector<float> &alphas_prev,
                               const std::vector<float> &sqrt_one_minus_alphas, DeviceBuffer &e_t) {
    const int rc = apply_model(x, t, c, e_t);
    if (rc != 0) return rc;
    return msd_ddim_update(x.ptr(), e_t.ptr(), x.ptr(), x.count(), alphas[index], alphas_prev[index],
                           sqrt_one_minus_alphas[index], (int)x.dtype(), stream);
}

}  // namespace msd
