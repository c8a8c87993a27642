// C ABI of libmsd_hip.so (declared in include/msd_hip.h): argument checks, dtype
// dispatch and the per-(device, stream) GroupNorm scratch.
#include <cmath>
#include <mutex>
#include <unordered_map>

#include <hip/hip_fp16.h>

#include "msd_internal.h"

namespace msd {
namespace {

struct ScratchKey {
    int device;
    hipStream_t stream;
    bool operator==(const ScratchKey &o) const { return device == o.device && stream == o.stream; }
};
struct ScratchKeyHash {
    size_t operator()(const ScratchKey &k) const {
        return std::hash<void *>()((void *)k.stream) ^ (std::hash<int>()(k.device) * 0x9E3779B1u);
    }
};

std::mutex g_scratch_mutex;
std::unordered_map<ScratchKey, GnScratch, ScratchKeyHash> g_scratch;

// Scratch for `units` (sample, group) pairs, carved out of one block:
// [slot_mean | slot_m2 | epoch | done | fallbacks], every part 256-byte aligned.
constexpr size_t slot_bytes(size_t units) { return sizeof(unsigned long long) * units * kGnMaxSplit; }
constexpr size_t word_bytes(size_t units) { return sizeof(uint32_t) * units; }
constexpr size_t scratch_bytes(size_t units) { return 2 * slot_bytes(units) + 2 * word_bytes(units) + 256; }

GnScratch carve(char *base, size_t units) {
    GnScratch s;
    s.slot_mean = reinterpret_cast<unsigned long long *>(base);
    s.slot_m2 = reinterpret_cast<unsigned long long *>(base + slot_bytes(units));
    s.epoch = reinterpret_cast<uint32_t *>(base + 2 * slot_bytes(units));
    s.done = reinterpret_cast<uint32_t *>(base + 2 * slot_bytes(units) + word_bytes(units));
    s.fallbacks = reinterpret_cast<uint32_t *>(base + 2 * slot_bytes(units) + 2 * word_bytes(units));
    s.units = (uint32_t)units;
    return s;
}

// Scratch of the entry point that allocates nothing: part of the code object, one copy per
// device, zero when the module is loaded (tags, launch counts and counters start at zero and
// are never reset: see groupnorm.hip).  In host code this name is only a handle for
// hipGetSymbolAddress; kernels get the device address that call returns.
constexpr uint32_t kStaticUnits = 1024;
static __device__ __align__(256) unsigned char scratch[scratch_bytes(kStaticUnits)];

constexpr int kMaxDevices = 64;
char *g_static_base[kMaxDevices] = {nullptr};  // device address of `scratch`, per device

}  // namespace

// Scratch is private to a (device, stream) pair: launches on one stream are ordered, so a
// unit's slots are never shared by two launches in flight.
hipError_t get_scratch(hipStream_t stream, GnScratch *out) {
    // one handle that names a different stream in every thread cannot key a per-stream scratch
    if (stream == hipStreamPerThread) return hipErrorInvalidValue;
    int device = 0;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return err;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    const ScratchKey key{device, stream};
    auto it = g_scratch.find(key);
    if (it != g_scratch.end()) {
        *out = it->second;
        return hipSuccess;
    }
    char *base = nullptr;
    err = hipMalloc(reinterpret_cast<void **>(&base), scratch_bytes(kGnMaxUnits));
    if (err != hipSuccess) return err;
    err = hipMemset(base, 0, scratch_bytes(kGnMaxUnits));  // tags, epochs and counters start at zero
    // the fill runs on the null stream: it must have finished before a launch on `stream`
    // (which may not synchronise with the null stream) reads the scratch
    if (err == hipSuccess) err = hipStreamSynchronize(nullptr);
    if (err != hipSuccess) {
        (void)hipFree(base);
        return err;
    }
    const GnScratch s = carve(base, kGnMaxUnits);
    g_scratch.emplace(key, s);
    *out = s;
    return hipSuccess;
}

// The device address of the static scratch on the current device, looked up once per device.
hipError_t get_static_scratch(GnScratch *out) {
    int device = 0;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return err;
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_static_base[device] == nullptr) {
        void *ptr = nullptr;
        err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess) return err;
        if (ptr == nullptr) return hipErrorInvalidSymbol;
        g_static_base[device] = static_cast<char *>(ptr);
    }
    *out = carve(g_static_base[device], kStaticUnits);
    return hipSuccess;
}

Tuning g_tuning{};

}  // namespace msd

using namespace msd;

extern "C" {

int msd_version(void) { return 200; }

const char *msd_error_string(int code) {
    if (code == MSD_OK) return "ok";
    if (code == MSD_ERR_INVALID_VALUE) return "invalid value (shape, pointer or dtype rejected)";
    if (code == MSD_ERR_SCRATCH_LIMIT)
        return "msd_groupnorm_noalloc: batch * groups exceeds the 1024 units its fixed scratch holds";
    return hipGetErrorString(static_cast<hipError_t>(code));
}

int msd_init(void *stream) {
    GnScratch sc;
    hipError_t err = get_static_scratch(&sc);
    if (err != hipSuccess) return (int)err;
    return (int)get_scratch(static_cast<hipStream_t>(stream), &sc);
}

int msd_release(void *stream) {
    int device = 0;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return (int)err;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    auto it = g_scratch.find(ScratchKey{device, static_cast<hipStream_t>(stream)});
    if (it == g_scratch.end()) return MSD_OK;
    err = hipFree(it->second.slot_mean);
    g_scratch.erase(it);
    return (int)err;
}

int msd_shutdown(void) {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    int rc = MSD_OK;
    int current = 0;
    (void)hipGetDevice(&current);
    for (auto &kv : g_scratch) {
        (void)hipSetDevice(kv.first.device);
        const hipError_t err = hipFree(kv.second.slot_mean);
        if (err != hipSuccess) rc = (int)err;
    }
    g_scratch.clear();
    (void)hipSetDevice(current);
    return rc;
}

int msd_status(void *stream) { return (int)hipStreamSynchronize(static_cast<hipStream_t>(stream)); }

int msd_gn_fallbacks(void *stream, unsigned int *count, int reset) {
    if (!count) return MSD_ERR_INVALID_VALUE;
    *count = 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t err = hipStreamSynchronize(s);
    if (err != hipSuccess) return (int)err;
    int device = 0;
    err = hipGetDevice(&device);
    if (err != hipSuccess) return (int)err;
    uint32_t *counters[2] = {nullptr, nullptr};
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        auto it = g_scratch.find(ScratchKey{device, s});
        if (it != g_scratch.end()) counters[0] = it->second.fallbacks;
        if (device >= 0 && device < kMaxDevices && g_static_base[device])
            counters[1] = carve(g_static_base[device], kStaticUnits).fallbacks;
    }
    for (uint32_t *c : counters) {
        if (!c) continue;
        uint32_t v = 0;
        err = hipMemcpy(&v, c, sizeof(v), hipMemcpyDeviceToHost);
        if (err != hipSuccess) return (int)err;
        *count += v;
        if (reset && v) {
            v = 0;
            err = hipMemcpy(c, &v, sizeof(v), hipMemcpyHostToDevice);
            if (err != hipSuccess) return (int)err;
        }
    }
    return MSD_OK;
}

int msd_set_tuning(int knob, int value) {
    if (value < 0) return MSD_ERR_INVALID_VALUE;
    switch (knob) {
        case MSD_TUNE_GN_SPLIT:
            if (value && ((value & (value - 1)) != 0 || value > (int)kGnMaxSplit)) return MSD_ERR_INVALID_VALUE;
            g_tuning.gn_split = value;
            return MSD_OK;
        case MSD_TUNE_GN_THREADS:
            if (value && (value % 64 != 0 || value > 1024)) return MSD_ERR_INVALID_VALUE;
            g_tuning.gn_threads = value;
            return MSD_OK;
        case MSD_TUNE_LN_CHUNK:
            if (value && value != 8 && value != 16) return MSD_ERR_INVALID_VALUE;
            g_tuning.ln_chunk = value;
            return MSD_OK;
        case MSD_TUNE_LN_THREADS:
            if (value && value != 64 && value != 128 && value != 256 && value != 512) return MSD_ERR_INVALID_VALUE;
            g_tuning.ln_threads = value;
            return MSD_OK;
        case MSD_TUNE_GEGLU_VECTORS:
            if (value && value != 1 && value != 2 && value != 4) return MSD_ERR_INVALID_VALUE;
            g_tuning.geglu_vectors = value;
            return MSD_OK;
        case MSD_TUNE_ACT_VECTORS:
            if (value && value != 1 && value != 2 && value != 4) return MSD_ERR_INVALID_VALUE;
            g_tuning.act_vectors = value;
            return MSD_OK;
        case MSD_TUNE_SOFTMAX_ROWS:
            if (value && value != 16 && value != 32 && value != 64) return MSD_ERR_INVALID_VALUE;
            g_tuning.softmax_rows = value;
            return MSD_OK;
        case MSD_TUNE_GN_SPIN_LIMIT:
            g_tuning.gn_spin_limit = value;
            return MSD_OK;
        case MSD_TUNE_GN_WRITERS:
            if (value && ((value & (value - 1)) != 0 || value > 16)) return MSD_ERR_INVALID_VALUE;
            g_tuning.gn_writers = value;
            return MSD_OK;
        case MSD_TUNE_DEVICE_CUS:
            if (value > 4096) return MSD_ERR_INVALID_VALUE;
            g_tuning.device_cus = value;
            return MSD_OK;
        case MSD_TUNE_DEVICE_XCDS:
            if (value > 64) return MSD_ERR_INVALID_VALUE;
            g_tuning.device_xcds = value;
            return MSD_OK;
        case MSD_TUNE_GN_PLAN_RULE_ONLY:
            if (value > 1) return MSD_ERR_INVALID_VALUE;
            g_tuning.gn_plan_rule_only = value;
            return MSD_OK;
        default:
            return MSD_ERR_INVALID_VALUE;
    }
}

// Byte ranges [a, a + abytes) and [b, b + bbytes) share at least one byte.
static bool ranges_overlap(const void *a, size_t abytes, const void *b, size_t bbytes) {
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
    return abytes != 0 && bbytes != 0 && a0 < b0 + bbytes && b0 < a0 + abytes;
}
// An output that may take the place of its input must be exactly that input or lie apart from
// it: a shifted overlap would let one workgroup store into what another still has to load.
static bool shifted_overlap(const void *in, const void *out, size_t bytes) {
    return in != out && ranges_overlap(in, bytes, out, bytes);
}
static size_t elt_bytes(int dtype) { return dtype == MSD_DTYPE_F32 ? 4 : 2; }

static int groupnorm_entry(const void *x, const void *chunk, void *y, const float *gamma,
                           const float *beta, size_t batch, size_t channels, size_t hw, size_t groups,
                           float eps, int fuse_silu, int dtype, const GnScratch *fixed, void *stream) {
    if (groups == 0 || channels == 0 || channels % groups != 0) return MSD_ERR_INVALID_VALUE;
    if (dtype != MSD_DTYPE_F32 && dtype != MSD_DTYPE_F16) return MSD_ERR_INVALID_VALUE;
    if (batch * hw != 0 && (!x || !y || !gamma || !beta)) return MSD_ERR_INVALID_VALUE;
    size_t count;
    if (__builtin_mul_overflow(batch, channels, &count) || __builtin_mul_overflow(count, hw, &count) ||
        count > (SIZE_MAX >> 3))
        return MSD_ERR_INVALID_VALUE;
    if (shifted_overlap(x, y, count * elt_bytes(dtype))) return MSD_ERR_INVALID_VALUE;
    // the addend is read by every workgroup of its (sample, channel) while others already store
    if (chunk != nullptr && ranges_overlap(chunk, batch * channels * elt_bytes(dtype), y, count * elt_bytes(dtype)))
        return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // Whether a launch needs the per-stream scratch depends on its shape; the rule does not:
    // the one handle that names a different stream in every thread is refused for every call
    // that may use that scratch (msd_groupnorm_noalloc, which has its own, takes it).
    if (fixed == nullptr && s == hipStreamPerThread) return MSD_ERR_INVALID_VALUE;
    if (dtype == MSD_DTYPE_F32)
        return gn_dispatch<float>(x, chunk, y, gamma, beta, batch, channels, hw, groups, eps,
                                  fuse_silu != 0, fixed, s);
    return gn_dispatch<__half>(x, chunk, y, gamma, beta, batch, channels, hw, groups, eps,
                               fuse_silu != 0, fixed, s);
}

int msd_groupnorm(const void *x, void *y, const float *gamma, const float *beta, size_t batch,
                  size_t channels, size_t hw, size_t groups, float eps, int fuse_silu, int dtype,
                  void *stream) {
    return groupnorm_entry(x, nullptr, y, gamma, beta, batch, channels, hw, groups, eps, fuse_silu,
                           dtype, nullptr, stream);
}

int msd_groupnorm_plan(size_t batch, size_t channels, size_t hw, size_t groups, int dtype, int noalloc,
                       int in_place, int *split, int *threads, int *vectors_per_lane, int *writers) {
    if (!split || !threads || !vectors_per_lane || !writers) return MSD_ERR_INVALID_VALUE;
    if (groups == 0 || channels == 0 || channels % groups != 0) return MSD_ERR_INVALID_VALUE;
    if (dtype != MSD_DTYPE_F32 && dtype != MSD_DTYPE_F16) return MSD_ERR_INVALID_VALUE;
    if (batch * groups > 0x7FFFFFFFull || (channels / groups) * hw > 0x7FFFFFFFull) return MSD_ERR_INVALID_VALUE;
    if (noalloc && batch * groups > kStaticUnits) return MSD_ERR_SCRATCH_LIMIT;
    GnDecision d{0, 0, 0, 0, 1};
    if (batch * hw != 0)
        d = gn_decide(dtype == MSD_DTYPE_F32 ? 4 : 2, batch, channels, hw, groups, true,
                      noalloc ? (size_t)kStaticUnits : (size_t)kGnMaxUnits, in_place == 0);
    *split = (int)d.split;
    *threads = (int)d.threads;
    *vectors_per_lane = (int)d.k;
    *writers = (int)d.writers;
    return MSD_OK;
}

int msd_groupnorm_noalloc(const void *x, void *y, const float *gamma, const float *beta, size_t batch,
                          size_t channels, size_t hw, size_t groups, float eps, int fuse_silu, int dtype,
                          void *stream) {
    // the size check comes first so that it does not depend on a device being present
    if (batch > kStaticUnits || groups > kStaticUnits || batch * groups > kStaticUnits)
        return MSD_ERR_SCRATCH_LIMIT;
    GnScratch fixed;
    const hipError_t err = get_static_scratch(&fixed);  // a table lookup after the first call on a device
    if (err != hipSuccess) return (int)err;
    return groupnorm_entry(x, nullptr, y, gamma, beta, batch, channels, hw, groups, eps, fuse_silu,
                           dtype, &fixed, stream);
}

int msd_chunk_add_groupnorm(const void *x, const void *chunk, void *y, const float *gamma,
                            const float *beta, size_t batch, size_t channels, size_t hw,
                            size_t groups, float eps, int fuse_silu, int dtype, void *stream) {
    if (batch * hw != 0 && !chunk) return MSD_ERR_INVALID_VALUE;
    return groupnorm_entry(x, chunk, y, gamma, beta, batch, channels, hw, groups, eps, fuse_silu,
                           dtype, nullptr, stream);
}

int msd_groupnorm_tokens(const void *x, void *y, const float *gamma, const float *beta, size_t batch,
                         size_t channels, size_t hw, size_t groups, float eps, int dtype,
                         void *stream) {
    if (groups == 0 || channels == 0 || channels % groups != 0) return MSD_ERR_INVALID_VALUE;
    if (dtype != MSD_DTYPE_F32 && dtype != MSD_DTYPE_F16) return MSD_ERR_INVALID_VALUE;
    if (batch * hw != 0 && (!x || !y || !gamma || !beta)) return MSD_ERR_INVALID_VALUE;
    size_t count;
    if (__builtin_mul_overflow(batch, channels, &count) || __builtin_mul_overflow(count, hw, &count) ||
        count > (SIZE_MAX >> 3))
        return MSD_ERR_INVALID_VALUE;
    if (ranges_overlap(x, count * elt_bytes(dtype), y, count * elt_bytes(dtype))) return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (s == hipStreamPerThread) return MSD_ERR_INVALID_VALUE;  // as for msd_groupnorm: may need the per-stream scratch
    if (dtype == MSD_DTYPE_F32)
        return gn_tokens_dispatch<float>(x, y, gamma, beta, batch, channels, hw, groups, eps, s);
    return gn_tokens_dispatch<__half>(x, y, gamma, beta, batch, channels, hw, groups, eps, s);
}

static int layernorm_entry(const void *x, const void *res, void *sum, void *y, const float *gamma,
                           const float *beta, size_t rows, size_t dim, float eps, int dtype,
                           void *stream) {
    if (dtype != MSD_DTYPE_F32 && dtype != MSD_DTYPE_F16) return MSD_ERR_INVALID_VALUE;
    if (rows * dim != 0 && (!x || !y || !gamma || !beta)) return MSD_ERR_INVALID_VALUE;
    size_t count;
    if (__builtin_mul_overflow(rows, dim, &count) || count > (SIZE_MAX >> 3)) return MSD_ERR_INVALID_VALUE;
    const size_t bytes = count * elt_bytes(dtype);
    if (shifted_overlap(x, y, bytes)) return MSD_ERR_INVALID_VALUE;
    if (res != nullptr && (shifted_overlap(x, sum, bytes) || shifted_overlap(res, sum, bytes) ||
                           ranges_overlap(sum, bytes, y, bytes) || shifted_overlap(res, y, bytes)))
        return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MSD_DTYPE_F32)
        return ln_dispatch<float>(x, res, sum, y, gamma, beta, rows, dim, eps, s);
    return ln_dispatch<__half>(x, res, sum, y, gamma, beta, rows, dim, eps, s);
}

int msd_layernorm(const void *x, void *y, const float *gamma, const float *beta, size_t rows,
                  size_t dim, float eps, int dtype, void *stream) {
    return layernorm_entry(x, nullptr, nullptr, y, gamma, beta, rows, dim, eps, dtype, stream);
}

int msd_add_layernorm(const void *a, const void *b, void *sum, void *y, const float *gamma,
                      const float *beta, size_t rows, size_t dim, float eps, int dtype,
                      void *stream) {
    if (rows * dim != 0 && (!b || !sum)) return MSD_ERR_INVALID_VALUE;
    return layernorm_entry(a, b, sum, y, gamma, beta, rows, dim, eps, dtype, stream);
}

int msd_elemwise_add(const void *a, const void *b, void *c, size_t n, int dtype, void *stream) {
    if (dtype != MSD_DTYPE_F32 && dtype != MSD_DTYPE_F16) return MSD_ERR_INVALID_VALUE;
    if (n != 0 && (!a || !b || !c)) return MSD_ERR_INVALID_VALUE;
    if (n > (SIZE_MAX >> 3)) return MSD_ERR_INVALID_VALUE;
    if (shifted_overlap(a, c, n * elt_bytes(dtype)) || shifted_overlap(b, c, n * elt_bytes(dtype)))
        return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MSD_DTYPE_F32) return add_dispatch<float>(a, b, c, n, 0, s);
    return add_dispatch<__half>(a, b, c, n, 0, s);
}

int msd_chunkwise_add(const void *a, const void *chunk, void *c, size_t n, size_t chunk_size,
                      int dtype, void *stream) {
    if (dtype != MSD_DTYPE_F32 && dtype != MSD_DTYPE_F16) return MSD_ERR_INVALID_VALUE;
    if (chunk_size == 0) return MSD_ERR_INVALID_VALUE;
    if (n != 0 && (!a || !chunk || !c)) return MSD_ERR_INVALID_VALUE;
    if (n > (SIZE_MAX >> 3)) return MSD_ERR_INVALID_VALUE;
    if (shifted_overlap(a, c, n * elt_bytes(dtype)) ||
        ranges_overlap(chunk, (n / chunk_size) * elt_bytes(dtype), c, n * elt_bytes(dtype)))
        return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MSD_DTYPE_F32) return add_dispatch<float>(a, chunk, c, n, chunk_size, s);
    return add_dispatch<__half>(a, chunk, c, n, chunk_size, s);
}

int msd_geglu(const void *proj, void *out, size_t rows, size_t inner, int dtype, void *stream) {
    if (dtype != MSD_DTYPE_F32 && dtype != MSD_DTYPE_F16) return MSD_ERR_INVALID_VALUE;
    if (rows * inner != 0 && (!proj || !out)) return MSD_ERR_INVALID_VALUE;
    size_t count;
    if (__builtin_mul_overflow(rows, inner, &count) || count > (SIZE_MAX >> 4)) return MSD_ERR_INVALID_VALUE;
    // rows of proj and out have different strides: an overlapping out would be read after it was written
    if (ranges_overlap(proj, 2 * count * elt_bytes(dtype), out, count * elt_bytes(dtype))) return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MSD_DTYPE_F32) return geglu_dispatch<float>(proj, out, rows, inner, s);
    return geglu_dispatch<__half>(proj, out, rows, inner, s);
}

static int act_entry(Act op, const void *x, void *y, size_t n, int dtype, void *stream) {
    if (dtype != MSD_DTYPE_F32 && dtype != MSD_DTYPE_F16) return MSD_ERR_INVALID_VALUE;
    if (n != 0 && (!x || !y)) return MSD_ERR_INVALID_VALUE;
    if (n > (SIZE_MAX >> 3) || shifted_overlap(x, y, n * elt_bytes(dtype))) return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MSD_DTYPE_F32) return act_dispatch<float>(op, x, y, n, s);
    return act_dispatch<__half>(op, x, y, n, s);
}

int msd_silu(const void *x, void *y, size_t n, int dtype, void *stream) {
    return act_entry(Act::Silu, x, y, n, dtype, stream);
}
int msd_gelu(const void *x, void *y, size_t n, int dtype, void *stream) {
    return act_entry(Act::Gelu, x, y, n, dtype, stream);
}
int msd_quick_gelu(const void *x, void *y, size_t n, int dtype, void *stream) {
    return act_entry(Act::QuickGelu, x, y, n, dtype, stream);
}

int msd_permute_0_2_1(const void *src, void *dst, size_t isize, size_t jsize, size_t ksize, int dtype,
                      void *stream) {
    if (dtype != MSD_DTYPE_F32 && dtype != MSD_DTYPE_F16) return MSD_ERR_INVALID_VALUE;
    if (isize * jsize * ksize != 0 && (!src || !dst)) return MSD_ERR_INVALID_VALUE;
    size_t count;
    if (__builtin_mul_overflow(isize, jsize, &count) || __builtin_mul_overflow(count, ksize, &count) ||
        count > (SIZE_MAX >> 3))
        return MSD_ERR_INVALID_VALUE;
    if (ranges_overlap(src, count * elt_bytes(dtype), dst, count * elt_bytes(dtype))) return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MSD_DTYPE_F32) return permute_021_dispatch<float>(src, dst, isize, jsize, ksize, s);
    return permute_021_dispatch<__half>(src, dst, isize, jsize, ksize, s);
}

int msd_copy(const void *src, void *dst, size_t bytes, void *stream) {
    if (bytes % 4 != 0) return MSD_ERR_INVALID_VALUE;
    return act_entry(Act::Copy, src, dst, bytes / 4, MSD_DTYPE_F32, stream);
}

int msd_timestep_embedding(const int64_t *timesteps, void *out, size_t batch, size_t dim,
                           float max_period, int dtype, void *stream) {
    if (dim % 2 != 0 || !(max_period > 0.0f)) return MSD_ERR_INVALID_VALUE;
    if (dtype != MSD_DTYPE_F32 && dtype != MSD_DTYPE_F16) return MSD_ERR_INVALID_VALUE;
    if (batch * dim == 0) return MSD_OK;
    if (!timesteps || !out || batch * dim > 0x7FFFFFFFull) return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MSD_DTYPE_F32)
        return temb_dispatch<float>(timesteps, out, batch, dim, max_period, s);
    return temb_dispatch<__half>(timesteps, out, batch, dim, max_period, s);
}

int msd_ddim_timesteps(int ddim_num_steps, int *out, int cap) {
    const int ddpm_steps = 1000;
    if (ddim_num_steps < 1 || ddim_num_steps > ddpm_steps) return -1;
    const int stride = ddpm_steps / ddim_num_steps;
    int count = 0;
    for (int t = 1; t <= ddpm_steps; t += stride) {
        if (out && count < cap) out[count] = t;
        count++;
    }
    return count;
}

int msd_linear_rows(const void *x, const void *weight, const float *bias, void *y, size_t m,
                    size_t n, size_t k, int act_in, int act_out, int dtype, void *stream) {
    if (dtype != MSD_DTYPE_F32 && dtype != MSD_DTYPE_F16) return MSD_ERR_INVALID_VALUE;
    if ((act_in != MSD_ACT_NONE && act_in != MSD_ACT_SILU) ||
        (act_out != MSD_ACT_NONE && act_out != MSD_ACT_SILU))
        return MSD_ERR_INVALID_VALUE;
    if (m > 8) return MSD_ERR_INVALID_VALUE;
    if (m * n != 0 && (!y || (k != 0 && (!x || !weight)))) return MSD_ERR_INVALID_VALUE;
    if (n > (SIZE_MAX >> 8) || k > (SIZE_MAX >> 8)) return MSD_ERR_INVALID_VALUE;
    if (ranges_overlap(x, m * k * elt_bytes(dtype), y, m * n * elt_bytes(dtype))) return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MSD_DTYPE_F32)
        return linear_rows_dispatch<float>(x, weight, bias, y, m, n, k, act_in, act_out, s);
    return linear_rows_dispatch<__half>(x, weight, bias, y, m, n, k, act_in, act_out, s);
}

int msd_linear_rows_grouped(const void *x, const void *const *weights, const float *const *biases,
                            void *const *ys, const size_t *ns, size_t count, size_t m, size_t k,
                            int act_in, int act_out, int dtype, void *stream) {
    if (dtype != MSD_DTYPE_F32 && dtype != MSD_DTYPE_F16) return MSD_ERR_INVALID_VALUE;
    if ((act_in != MSD_ACT_NONE && act_in != MSD_ACT_SILU) ||
        (act_out != MSD_ACT_NONE && act_out != MSD_ACT_SILU))
        return MSD_ERR_INVALID_VALUE;
    if (m > 8) return MSD_ERR_INVALID_VALUE;
    if (count != 0 && (!weights || !ys || !ns)) return MSD_ERR_INVALID_VALUE;
    constexpr size_t kMaxExtent = (size_t)1 << 28;  // keeps every byte count below far inside size_t
    if (k > kMaxExtent) return MSD_ERR_INVALID_VALUE;
    for (size_t i = 0; i < count && m != 0; i++) {
        if (ns[i] == 0) continue;
        if (!ys[i] || (k != 0 && (!x || !weights[i])) || ns[i] > kMaxExtent) return MSD_ERR_INVALID_VALUE;
    }
    // the problems run side by side in one launch: no output may lie in the shared rows or in
    // any problem's output, weights or bias
    const size_t elt = elt_bytes(dtype);
    for (size_t i = 0; i < count && m != 0; i++) {
        if (ns[i] == 0) continue;
        const size_t ybytes = m * ns[i] * elt;
        if (ranges_overlap(x, m * k * elt, ys[i], ybytes)) return MSD_ERR_INVALID_VALUE;
        for (size_t j = 0; j < count; j++) {
            if (ns[j] == 0) continue;
            if (j != i && ranges_overlap(ys[j], m * ns[j] * elt, ys[i], ybytes)) return MSD_ERR_INVALID_VALUE;
            if (k != 0 && ranges_overlap(weights[j], ns[j] * k * elt, ys[i], ybytes)) return MSD_ERR_INVALID_VALUE;
            if (biases && biases[j] && ranges_overlap(biases[j], ns[j] * sizeof(float), ys[i], ybytes))
                return MSD_ERR_INVALID_VALUE;
        }
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MSD_DTYPE_F32)
        return linear_rows_grouped_dispatch<float>(x, weights, biases, ys, ns, count, m, k, act_in, act_out, s);
    return linear_rows_grouped_dispatch<__half>(x, weights, biases, ys, ns, count, m, k, act_in, act_out, s);
}

int msd_softmax(const void *x, void *y, size_t rows, size_t cols, int stable, int dtype,
                void *stream) {
    if (dtype != MSD_DTYPE_F32 && dtype != MSD_DTYPE_F16) return MSD_ERR_INVALID_VALUE;
    if (rows * cols != 0 && (!x || !y)) return MSD_ERR_INVALID_VALUE;
    size_t count;
    if (__builtin_mul_overflow(rows, cols, &count) || count > (SIZE_MAX >> 3)) return MSD_ERR_INVALID_VALUE;
    if (shifted_overlap(x, y, count * elt_bytes(dtype))) return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MSD_DTYPE_F32) return softmax_dispatch<float>(x, y, rows, cols, stable != 0, s);
    return softmax_dispatch<__half>(x, y, rows, cols, stable != 0, s);
}

int msd_alphas_cumprod(float *out_1000) {
    if (!out_1000) return MSD_ERR_INVALID_VALUE;
    const int steps = 1000;
    const double linear_start = 0.00085, linear_end = 0.0120;
    const double first = std::sqrt(linear_start), last = std::sqrt(linear_end);
    const double spacing = (last - first) / static_cast<double>(steps - 1);
    double product = 1.0;
    for (int i = 0; i < steps; i++) {
        const double root = first + static_cast<double>(i) * spacing;
        product *= 1.0 - root * root;
        out_1000[i] = static_cast<float>(product);
    }
    return MSD_OK;
}

int msd_ddim_schedule(int ddim_num_steps, int *timesteps, float *alphas, float *alphas_prev,
                      float *sqrt_one_minus_alphas, int cap) {
    static float cumprod[1000];
    static std::once_flag once;
    std::call_once(once, [] { (void)msd_alphas_cumprod(cumprod); });
    int local[1001];
    const int count = msd_ddim_timesteps(ddim_num_steps, local, 1001);
    if (count < 0) return -1;
    if (local[count - 1] >= 1000) return -2;
    for (int i = 0; i < count && i < cap; i++) {
        const float a = cumprod[local[i]];
        if (timesteps) timesteps[i] = local[i];
        if (alphas) alphas[i] = a;
        if (alphas_prev) alphas_prev[i] = i == 0 ? cumprod[0] : cumprod[local[i - 1]];
        if (sqrt_one_minus_alphas) sqrt_one_minus_alphas[i] = std::sqrt(1.0f - a);
    }
    return count;
}

int msd_ddim_update(const void *x, const void *e_t, void *x_prev, size_t n, float a_t,
                    float a_prev, float sqrt_one_minus_at, int dtype, void *stream) {
    if (dtype != MSD_DTYPE_F32 && dtype != MSD_DTYPE_F16) return MSD_ERR_INVALID_VALUE;
    if (n != 0 && (!x || !e_t || !x_prev)) return MSD_ERR_INVALID_VALUE;
    if (!(a_t > 0.0f) || !(a_prev >= 0.0f) || !(a_prev <= 1.0f)) return MSD_ERR_INVALID_VALUE;  // sqrt / division
    if (n > (SIZE_MAX >> 3) || shifted_overlap(x, x_prev, n * elt_bytes(dtype)) ||
        shifted_overlap(e_t, x_prev, n * elt_bytes(dtype)))
        return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MSD_DTYPE_F32)
        return ddim_update_dispatch<float>(x, e_t, x_prev, n, a_t, a_prev, sqrt_one_minus_at, s);
    return ddim_update_dispatch<__half>(x, e_t, x_prev, n, a_t, a_prev, sqrt_one_minus_at, s);
}

}  // extern "C"
