#include "util.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <stdexcept>

namespace msd {

DeviceBuffer DeviceBuffer::allocate(size_t bytes, DType dtype) {
    DeviceBuffer b;
    if (bytes) {
        const hipError_t err = hipMalloc(&b.ptr_, bytes);
        if (err != hipSuccess)
            throw std::runtime_error(std::string("hipMalloc failed: ") + hipGetErrorString(err));
    }
    b.bytes_ = bytes;
    b.dtype_ = dtype;
    b.owned_ = true;
    return b;
}

DeviceBuffer &DeviceBuffer::operator=(DeviceBuffer &&o) noexcept {
    if (this != &o) {
        release();
        ptr_ = o.ptr_;
        bytes_ = o.bytes_;
        dtype_ = o.dtype_;
        owned_ = o.owned_;
        o.ptr_ = nullptr;
        o.bytes_ = 0;
        o.owned_ = false;
    }
    return *this;
}

void DeviceBuffer::release() {
    if (owned_ && ptr_) (void)hipFree(ptr_);
    ptr_ = nullptr;
    bytes_ = 0;
    owned_ = false;
}

DeviceBuffer::~DeviceBuffer() { release(); }

namespace util {
namespace {
std::string g_media_path;
bool g_media_path_set = false;

// IEEE binary16 <-> binary32 on the host (round to nearest even), for fp16-storage buffers
uint16_t float_to_half(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u, absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) return (uint16_t)(sign | 0x7C00u | (absx > 0x7F800000u ? 0x0200u : 0u));
    if (absx >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);
    if (absx < 0x33000001u) return (uint16_t)sign;
    const int exp = (int)(absx >> 23) - 127;
    const uint32_t man = (absx & 0x007FFFFFu) | 0x00800000u;
    const int shift = exp < -14 ? 13 + (-14 - exp) : 13;
    const uint32_t hexp = exp < -14 ? 0u : (uint32_t)(exp + 15);
    uint32_t kept = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (kept & 1u))) kept++;
    return (uint16_t)(sign | ((hexp << 10) + kept - (hexp ? 0x400u : 0u)));
}

float half_to_float(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16, exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
    uint32_t x;
    if (exp == 0) {
        const float v = (float)man * 5.9604644775390625e-8f;
        memcpy(&x, &v, 4);
        x |= sign;
    } else if (exp == 31) {
        x = sign | 0x7F800000u | (man << 13);
    } else {
        x = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}
}  // namespace

void setMediaPath(const std::string &dir) {
    g_media_path = dir;
    if (!g_media_path.empty() && g_media_path.back() != '/') g_media_path += '/';
    g_media_path_set = true;
}

std::string mediaPath() {
    if (g_media_path_set) return g_media_path;
    const char *env = std::getenv("MSD_MEDIA_PATH");
    if (env && *env) {
        std::string p(env);
        if (p.back() != '/') p += '/';
        return p;
    }
    return "./";
}

npy::Array load_npy_file(const std::string &filename) { return npy::load(mediaPath() + filename); }

DeviceBuffer upload(const std::vector<float> &data, DType dtype, hipStream_t stream) {
    DeviceBuffer buf = DeviceBuffer::allocate(data.size() * dtype_size(dtype), dtype);
    if (data.empty()) return buf;
    hipError_t err;
    if (dtype == DType::F32) {
        err = hipMemcpyAsync(buf.ptr(), data.data(), buf.bytes(), hipMemcpyHostToDevice, stream);
        if (err == hipSuccess) err = hipStreamSynchronize(stream);
    } else {
        std::vector<uint16_t> h(data.size());
        for (size_t i = 0; i < data.size(); i++) h[i] = float_to_half(data[i]);
        err = hipMemcpyAsync(buf.ptr(), h.data(), buf.bytes(), hipMemcpyHostToDevice, stream);
        if (err == hipSuccess) err = hipStreamSynchronize(stream);
    }
    if (err != hipSuccess)
        throw std::runtime_error(std::string("upload failed: ") + hipGetErrorString(err));
    return buf;
}

std::vector<float> download(const DeviceBuffer &buffer, hipStream_t stream) {
    std::vector<float> out(buffer.count());
    if (out.empty()) return out;
    hipError_t err;
    if (buffer.dtype() == DType::F32) {
        err = hipMemcpyAsync(out.data(), buffer.ptr(), buffer.bytes(), hipMemcpyDeviceToHost, stream);
        if (err == hipSuccess) err = hipStreamSynchronize(stream);
    } else {
        std::vector<uint16_t> h(out.size());
        err = hipMemcpyAsync(h.data(), buffer.ptr(), buffer.bytes(), hipMemcpyDeviceToHost, stream);
        if (err == hipSuccess) err = hipStreamSynchronize(stream);
        for (size_t i = 0; i < out.size(); i++) out[i] = half_to_float(h[i]);
    }
    if (err != hipSuccess)
        throw std::runtime_error(std::string("download failed: ") + hipGetErrorString(err));
    return out;
}

DeviceBuffer load_npy_file(const std::string &filename, size_t *num_vals, hipStream_t stream) {
    const npy::Array arr = load_npy_file(filename);
    if (num_vals) *num_vals = arr.num_vals();
    return upload(arr.data, DType::F32, stream);
}

TestResult testBuffer(const std::vector<float> &result, const char *filename) {
    TestResult r;
    const npy::Array test = load_npy_file(filename);
    if (result.size() != test.num_vals()) {
        fprintf(stderr, "%s: bufferSize(%zu) != test.num_vals(%zu)\n", filename, result.size(),
                test.num_vals());
        return r;
    }
    r.size_matches = true;
    for (size_t i = 0; i < result.size(); i++) {
        if (result[i] != test.data[i]) {
            r.num_wrong++;
            const float diff = std::fabs(result[i] - test.data[i]);
            if (diff > r.max_diff || std::isnan(diff)) {
                r.max_diff = diff;
                r.max_id = i;
            }
        }
    }
    if (!result.empty())
        fprintf(stderr, "%s max diff: %.20f / num : %zu / result[%zu]: %f/ test[%zu]: %f\n", filename,
                r.max_diff, r.num_wrong, r.max_id, result[r.max_id], r.max_id, test.data[r.max_id]);
    return r;
}

TestResult testBuffer(hipStream_t stream, const DeviceBuffer &buffer, const char *filename) {
    return testBuffer(download(buffer, stream), filename);
}

float printEventTime(const std::string &message, hipEvent_t start, hipEvent_t stop) {
    float ms = -1.0f;
    if (hipEventSynchronize(stop) != hipSuccess || hipEventElapsedTime(&ms, start, stop) != hipSuccess)
        return -1.0f;
    fprintf(stderr, "%s, %0.3f\n", message.c_str(), ms);
    return ms;
}

namespace {
int g_debug_timing = -1;  // -1: not decided yet (environment), 0 off, 1 on
}

void setDebugTiming(bool on) { g_debug_timing = on ? 1 : 0; }

bool debugTiming() {
    if (g_debug_timing < 0) {
        const char *env = getenv("MSD_DEBUG_TIMING");
        g_debug_timing = (env && env[0] && env[0] != '0') ? 1 : 0;
    }
    return g_debug_timing == 1;
}

LaunchTimer::LaunchTimer(hipStream_t stream) : stream_(stream) {
    if (!debugTiming()) return;
    // no timing inside a stream capture: waiting for an event there would invalidate it
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream_, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) return;
    if (hipEventCreate(&start_) != hipSuccess || hipEventCreate(&stop_) != hipSuccess ||
        hipEventRecord(start_, stream_) != hipSuccess) {
        if (start_) (void)hipEventDestroy(start_);
        if (stop_) (void)hipEventDestroy(stop_);
        start_ = stop_ = nullptr;
    }
}

LaunchTimer::~LaunchTimer() {
    if (start_) (void)hipEventDestroy(start_);
    if (stop_) (void)hipEventDestroy(stop_);
}

float LaunchTimer::finish(const std::string &message) {
    if (!start_ || !stop_) return -1.0f;
    if (hipEventRecord(stop_, stream_) != hipSuccess) return -1.0f;
    return printEventTime(message, start_, stop_);
}

}  // namespace util
}  // namespace msd
