// gfx950 kernels and C ABI for the norm / activation / embedding path.
//
// All kernels are bandwidth-bound streaming or reduction kernels: 16-byte
// coalesced loads issued up front, float32 arithmetic, 64-wide DPP reductions,
// no matrix cores.  Storage is float32 or binary16 (template parameter T).
//
// GroupNorm(+SiLU)   gn_split_kernel : S workgroups share one (sample, group)
//                    unit; each keeps its slice in registers (one HBM read),
//                    slices exchange (mean, M2) through device memory and
//                    combine them with Chan's formula, then normalise from
//                    registers (one HBM write).
// LayerNorm          ln_team_kernel  : a row is owned by a team of TL lanes of
//                    one wavefront, VPL 16-byte vectors per lane, two-pass
//                    statistics in registers.
// GEGLU / SiLU / GELU / quick_GELU : flat streaming kernels, U vectors per lane.
// Timestep embedding : one lane per (sample, frequency), frequency and angle
//                    rounded exactly as the float32 host loop it replaces.
#include "msd_device.h"

#include <mutex>
#include <unordered_map>
#include <vector>

#include "../../include/msd_hip.h"

using namespace msd;

namespace {

// ===========================================================================
// GroupNorm
// ===========================================================================
constexpr int kGnThreads = 256;           // workgroup size of gn_split_kernel
constexpr int kGnMaxSplit = 64;           // max workgroups per unit (one wavefront reads them)
constexpr uint32_t kGnEpoch = 64;         // arrival counter advances by this per launch per unit
constexpr uint32_t kGnMaxUnits = 8192;    // units with scratch slots; more units never split
constexpr uint32_t kGnSpinLimit = 1u << 22;

struct GnScratch {
    unsigned long long *partial;  // [kGnMaxUnits][kGnMaxSplit] packed (mean, M2)
    uint32_t *counter;            // [kGnMaxUnits] arrival counters, never reset
    uint32_t *status;             // [1] sticky: bit 0 = a wait ran out of spins
};

struct GnParams {
    uint32_t vec_per_unit;   // 16-byte vectors per (sample, group)
    uint32_t vec_per_slice;  // vectors per workgroup (last slice may be shorter)
    uint32_t split;          // workgroups per unit, power of two <= kGnMaxSplit
    uint32_t split_shift;    // log2(split)
    uint32_t groups;
    uint32_t ch_per_group;
    FastDiv hw_vec;          // vectors per channel
    float eps;
    float inv_count;         // 1 / elements per unit
};

__device__ __forceinline__ unsigned long long pack_pair(float a, float b) {
    return (unsigned long long)__float_as_uint(a) |
           ((unsigned long long)__float_as_uint(b) << 32);
}

// One workgroup = one slice of one unit.  Workgroups of a unit have adjacent
// block ids, so every workgroup a waiter depends on was dispatched before or
// together with it; the wait is also bounded by kGnSpinLimit polls.
// FULL: every lane owns exactly K vectors (no masking anywhere).
template <typename T, int K, bool SILU, bool FULL>
__device__ __forceinline__ void gn_split_body(const T *x, T *y, const float *__restrict__ gamma,
                                              const float *__restrict__ beta,
                                              const GnScratch &scratch, const GnParams &p,
                                              uint32_t unit, uint32_t slice, uint32_t v_begin,
                                              uint32_t v_end, float *red_a, float *red_b,
                                              float *stats) {
    constexpr int EPV = Store<T>::EPV;
    constexpr int NW = kGnThreads / kWave;
    const uint32_t tid = threadIdx.x;
    const u32x4 *xin = reinterpret_cast<const u32x4 *>(x) + (size_t)unit * p.vec_per_unit;
    u32x4 *yout = reinterpret_cast<u32x4 *>(y) + (size_t)unit * p.vec_per_unit;

    // ---- the slice goes into registers: every load is issued before any use.
    // Lanes past the end of a ragged slice re-read its last vector (a valid
    // address) and zero it afterwards, so no load sits behind a branch.
    u32x4 raw[K];
    uint32_t vidx[K];
#pragma unroll
    for (int k = 0; k < K; k++) {
        const uint32_t v = v_begin + k * kGnThreads + tid;
        vidx[k] = FULL ? v : min(v, v_end - 1);
        raw[k] = load_stream(xin + vidx[k]);
    }
    // per-vector channel affine (gamma, beta), fetched while the data is in flight
    const uint32_t ch0 = (unit % p.groups) * p.ch_per_group;
    float ga[K], be[K];
#pragma unroll
    for (int k = 0; k < K; k++) {
        const uint32_t c = ch0 + fast_div(vidx[k], p.hw_vec);
        ga[k] = gamma[c];
        be[k] = beta[c];
    }

    // ---- slice mean
    float f[K][EPV];
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < K; k++) {
        if (!FULL) {
            const bool used = v_begin + k * kGnThreads + tid < v_end;
#pragma unroll
            for (int i = 0; i < 4; i++) raw[k][i] = used ? raw[k][i] : 0u;
        }
        Store<T>::unpack(raw[k], f[k]);
#pragma unroll
        for (int e = 0; e < EPV; e++) s += f[k][e];
    }
    const float slice_count = (float)((v_end - v_begin) * EPV);
    const float slice_mean = block_sum<NW>(s, red_a) / slice_count;

    // ---- slice M2 = sum (x - slice_mean)^2 over the slice only
    float q = 0.0f;
#pragma unroll
    for (int k = 0; k < K; k++) {
        float qk = 0.0f;
#pragma unroll
        for (int e = 0; e < EPV; e++) {
            const float d = f[k][e] - slice_mean;
            qk = fmaf(d, d, qk);
        }
        if (!FULL) qk = (v_begin + k * kGnThreads + tid < v_end) ? qk : 0.0f;
        q += qk;
    }
    const float slice_m2 = block_sum<NW>(q, red_b);

    float mean, rstd;
    if (p.split == 1) {
        mean = slice_mean;
        rstd = 1.0f / sqrtf(slice_m2 * p.inv_count + p.eps);
    } else {
        // ---- publish (mean, M2), wait for the other slices, combine
        unsigned long long *slots = scratch.partial + (size_t)unit * kGnMaxSplit;
        if (tid == 0) {
            __hip_atomic_store(slots + slice, pack_pair(slice_mean, slice_m2), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
            const uint32_t old =
                __hip_atomic_fetch_add(scratch.counter + unit, kGnEpoch >> p.split_shift,
                                       __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
            const uint32_t target = (old & ~(kGnEpoch - 1)) + kGnEpoch;
            uint32_t polls = 0;
            while ((int32_t)(__hip_atomic_load(scratch.counter + unit, __ATOMIC_ACQUIRE,
                                               __HIP_MEMORY_SCOPE_AGENT) -
                             target) < 0) {
                __builtin_amdgcn_s_sleep(1);
                if (++polls > kGnSpinLimit) {
                    __hip_atomic_fetch_or(scratch.status, 1u, __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
            }
        }
        __syncthreads();
        if (tid < kWave) {
            // lane l holds slice l (count n_l); Chan: M2 = sum M2_l + sum n_l (mean_l - mean)^2
            float m_l = 0.0f, q_l = 0.0f, n_l = 0.0f;
            if (tid < p.split) {
                const unsigned long long pr = __hip_atomic_load(
                    slots + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                m_l = __uint_as_float((uint32_t)pr);
                q_l = __uint_as_float((uint32_t)(pr >> 32));
                const uint32_t b = tid * p.vec_per_slice;
                const uint32_t e = min(p.vec_per_unit, b + p.vec_per_slice);
                n_l = (float)((e - b) * EPV);
            }
            const float total_mean = wave_sum(m_l * n_l) * p.inv_count;
            const float dm = m_l - total_mean;
            const float m2 = wave_sum(fmaf(n_l * dm, dm, q_l));
            if (tid == 0) {
                stats[0] = total_mean;
                stats[1] = 1.0f / sqrtf(m2 * p.inv_count + p.eps);
            }
        }
        __syncthreads();
        mean = stats[0];
        rstd = stats[1];
    }

    // ---- normalise from registers, per-channel affine, optional SiLU
#pragma unroll
    for (int k = 0; k < K; k++) {
        const float a = rstd * ga[k];
        float o[EPV];
#pragma unroll
        for (int e = 0; e < EPV; e++) {
            const float t = fmaf(f[k][e] - mean, a, be[k]);
            o[e] = SILU ? silu_f(t) : t;
        }
        const u32x4 packed = Store<T>::pack(o);
        if (FULL || v_begin + k * kGnThreads + tid < v_end) store_stream(yout + vidx[k], packed);
    }
}

template <typename T, int K, bool SILU>
__global__ __launch_bounds__(kGnThreads) void gn_split_kernel(
    const T *x, T *y, const float *__restrict__ gamma, const float *__restrict__ beta,
    GnScratch scratch, GnParams p) {
    constexpr int NW = kGnThreads / kWave;
    __shared__ float red_a[NW];
    __shared__ float red_b[NW];
    __shared__ float stats[2];
    const uint32_t unit = blockIdx.x >> p.split_shift;
    const uint32_t slice = blockIdx.x & (p.split - 1);
    const uint32_t v_begin = slice * p.vec_per_slice;
    const uint32_t v_end = min(p.vec_per_unit, v_begin + p.vec_per_slice);
    if (v_end - v_begin == K * kGnThreads)  // uniform over the workgroup
        gn_split_body<T, K, SILU, true>(x, y, gamma, beta, scratch, p, unit, slice, v_begin, v_end,
                                        red_a, red_b, stats);
    else
        gn_split_body<T, K, SILU, false>(x, y, gamma, beta, scratch, p, unit, slice, v_begin,
                                         v_end, red_a, red_b, stats);
}

// Any shape: one workgroup per unit, three passes over global memory with
// scalar accesses (the second and third pass hit in L2 for UNet-sized units).
template <typename T, bool SILU>
__global__ __launch_bounds__(kGnThreads) void gn_generic_kernel(
    const T *x, T *y, const float *__restrict__ gamma,
    const float *__restrict__ beta, uint32_t unit_size, uint32_t hw, uint32_t groups,
    uint32_t ch_per_group, float eps) {
    constexpr int NW = kGnThreads / kWave;
    __shared__ float red_a[NW];
    __shared__ float red_b[NW];
    const uint32_t unit = blockIdx.x;
    const T *xin = x + (size_t)unit * unit_size;
    T *yout = y + (size_t)unit * unit_size;
    float s = 0.0f;
    for (uint32_t i = threadIdx.x; i < unit_size; i += kGnThreads) s += Store<T>::load1(xin + i);
    const float mean = block_sum<NW>(s, red_a) / (float)unit_size;
    float q = 0.0f;
    for (uint32_t i = threadIdx.x; i < unit_size; i += kGnThreads) {
        const float d = Store<T>::load1(xin + i) - mean;
        q = fmaf(d, d, q);
    }
    const float rstd = 1.0f / sqrtf(block_sum<NW>(q, red_b) / (float)unit_size + eps);
    const uint32_t ch0 = (unit % groups) * ch_per_group;
    for (uint32_t i = threadIdx.x; i < unit_size; i += kGnThreads) {
        const uint32_t c = ch0 + i / hw;
        const float t = fmaf(Store<T>::load1(xin + i) - mean, rstd * gamma[c], beta[c]);
        Store<T>::store1(yout + i, SILU ? silu_f(t) : t);
    }
}

// ===========================================================================
// LayerNorm
// ===========================================================================
constexpr int kLnThreads = 256;

// A row of VPL*TL vectors is owned by TL adjacent lanes; a wavefront covers
// 64/TL consecutive rows.  Lane (team, j) loads vectors j, j+TL, ... of its row.
template <typename T, int VPL, int TL>
__global__ __launch_bounds__(kLnThreads) void ln_team_kernel(
    const T *x, T *y, const float *__restrict__ gamma,
    const float *__restrict__ beta, uint32_t rows, float eps, float inv_dim) {
    constexpr int EPV = Store<T>::EPV;
    constexpr int RPW = kWave / TL;  // rows per wavefront
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = blockIdx.x * (kLnThreads / kWave) + threadIdx.x / kWave;
    const uint32_t row = wave * RPW + lane / TL;
    const uint32_t j = lane % TL;
    const bool live = row < rows;
    // lanes past the last row re-read it (valid address, no branch around the loads)
    const size_t row_vec = (size_t)min(row, rows - 1) * (VPL * TL);
    const u32x4 *xin = reinterpret_cast<const u32x4 *>(x) + row_vec;
    u32x4 *yout = reinterpret_cast<u32x4 *>(y) + row_vec;

    u32x4 raw[VPL];
#pragma unroll
    for (int k = 0; k < VPL; k++) raw[k] = load_stream(xin + k * TL + j);
    float f[VPL][EPV];
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < VPL; k++) {
        Store<T>::unpack(raw[k], f[k]);
#pragma unroll
        for (int e = 0; e < EPV; e++) s += f[k][e];
    }
    const float mean = team_sum<TL>(s) * inv_dim;
    float q = 0.0f;
#pragma unroll
    for (int k = 0; k < VPL; k++)
#pragma unroll
        for (int e = 0; e < EPV; e++) {
            f[k][e] -= mean;
            q = fmaf(f[k][e], f[k][e], q);
        }
    const float rstd = 1.0f / sqrtf(team_sum<TL>(q) * inv_dim + eps);
    if (!live) return;
#pragma unroll
    for (int k = 0; k < VPL; k++) {
        const uint32_t col = (k * TL + j) * EPV;
        float o[EPV];
#pragma unroll
        for (int e4 = 0; e4 < EPV; e4 += 4) {
            const f32x4 g = *reinterpret_cast<const f32x4 *>(gamma + col + e4);
            const f32x4 b = *reinterpret_cast<const f32x4 *>(beta + col + e4);
#pragma unroll
            for (int e = 0; e < 4; e++) o[e4 + e] = fmaf(f[k][e4 + e] * rstd, g[e], b[e]);
        }
        store_stream(yout + k * TL + j, Store<T>::pack(o));
    }
}

// Any dim: one wavefront per row, scalar accesses, three passes.
template <typename T>
__global__ __launch_bounds__(kLnThreads) void ln_generic_kernel(
    const T *x, T *y, const float *__restrict__ gamma,
    const float *__restrict__ beta, uint32_t rows, uint32_t dim, float eps) {
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t row = blockIdx.x * (kLnThreads / kWave) + threadIdx.x / kWave;
    if (row >= rows) return;  // whole wavefront leaves together
    const T *xin = x + (size_t)row * dim;
    T *yout = y + (size_t)row * dim;
    float s = 0.0f;
    for (uint32_t i = lane; i < dim; i += kWave) s += Store<T>::load1(xin + i);
    const float mean = wave_sum(s) / (float)dim;
    float q = 0.0f;
    for (uint32_t i = lane; i < dim; i += kWave) {
        const float d = Store<T>::load1(xin + i) - mean;
        q = fmaf(d, d, q);
    }
    const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)dim + eps);
    for (uint32_t i = lane; i < dim; i += kWave) {
        const float t = (Store<T>::load1(xin + i) - mean) * rstd;
        Store<T>::store1(yout + i, fmaf(t, gamma[i], beta[i]));
    }
}

// ===========================================================================
// Streaming kernels: GEGLU and elementwise activations
// ===========================================================================
constexpr int kStreamThreads = 256;
constexpr int kStreamUnroll = 4;

// out[r, c] = proj[r, c] * gelu(proj[r, inner + c]); vectors never straddle a row.
// Every workgroup but the last takes the branch-free path: 2*U loads in flight
// per lane before the first use.
template <typename T>
__global__ __launch_bounds__(kStreamThreads) void geglu_kernel(const T *__restrict__ proj,
                                                               T *__restrict__ out,
                                                               uint32_t out_vecs,
                                                               FastDiv vec_per_row) {
    constexpr int EPV = Store<T>::EPV;
    constexpr int U = kStreamUnroll;
    const u32x4 *in = reinterpret_cast<const u32x4 *>(proj);
    u32x4 *o = reinterpret_cast<u32x4 *>(out);
    const uint32_t block_base = blockIdx.x * (kStreamThreads * U);
    const uint32_t base = block_base + threadIdx.x;
    const bool full = block_base + kStreamThreads * U <= out_vecs;  // uniform
    u32x4 va[U], vb[U];
    uint32_t ovs[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const uint32_t ov = base + u * kStreamThreads;
        ovs[u] = full ? ov : min(ov, out_vecs - 1);  // ragged last block re-reads the last vector
        const uint32_t r = fast_div(ovs[u], vec_per_row);
        const size_t iv = (size_t)ovs[u] + (size_t)r * vec_per_row.d;  // r*2*vpr + (ov - r*vpr)
        va[u] = load_stream(in + iv);
        vb[u] = load_stream(in + iv + vec_per_row.d);
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        float a[EPV], b[EPV], r[EPV];
        Store<T>::unpack(va[u], a);
        Store<T>::unpack(vb[u], b);
#pragma unroll
        for (int e = 0; e < EPV; e++) r[e] = a[e] * gelu_erf_f(b[e]);
        const u32x4 packed = Store<T>::pack(r);
        if (full || base + u * kStreamThreads < out_vecs) store_stream(o + ovs[u], packed);
    }
}

template <typename T>
__global__ __launch_bounds__(kStreamThreads) void geglu_generic_kernel(
    const T *__restrict__ proj, T *__restrict__ out, size_t rows, size_t inner) {
    const size_t n = rows * inner;
    for (size_t i = (size_t)blockIdx.x * kStreamThreads + threadIdx.x; i < n;
         i += (size_t)gridDim.x * kStreamThreads) {
        const size_t r = i / inner, c = i - r * inner;
        const float a = Store<T>::load1(proj + r * 2 * inner + c);
        const float b = Store<T>::load1(proj + r * 2 * inner + inner + c);
        Store<T>::store1(out + i, a * gelu_erf_f(b));
    }
}

// y[i] = OP(x[i]); y may alias x: a lane reads its vectors before it writes them,
// and in the ragged last block the duplicated reads are never written back.
template <typename T, typename OP>
__global__ __launch_bounds__(kStreamThreads) void act_kernel(const T *x, T *y, uint32_t vecs,
                                                             size_t n) {
    constexpr int EPV = Store<T>::EPV;
    constexpr int U = kStreamUnroll;
    const u32x4 *in = reinterpret_cast<const u32x4 *>(x);
    u32x4 *o = reinterpret_cast<u32x4 *>(y);
    const uint32_t block_base = blockIdx.x * (kStreamThreads * U);
    const uint32_t base = block_base + threadIdx.x;
    const bool full = block_base + kStreamThreads * U <= vecs;  // uniform
    if (vecs != 0) {
        u32x4 raw[U];
        uint32_t vs[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t v = base + u * kStreamThreads;
            vs[u] = full ? v : min(v, vecs - 1);
            raw[u] = load_stream(in + vs[u]);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            float f[EPV];
            Store<T>::unpack(raw[u], f);
#pragma unroll
            for (int e = 0; e < EPV; e++) f[e] = OP::apply(f[e]);
            const u32x4 packed = Store<T>::pack(f);
            if (full || base + u * kStreamThreads < vecs) store_stream(o + vs[u], packed);
        }
    }
    // ragged tail (n % EPV elements) by the first lanes of block 0
    const size_t tail = (size_t)vecs * EPV;
    if (blockIdx.x == 0 && tail + threadIdx.x < n)
        Store<T>::store1(y + tail + threadIdx.x,
                         OP::apply(Store<T>::load1(x + tail + threadIdx.x)));
}

template <typename T, typename OP>
__global__ __launch_bounds__(kStreamThreads) void act_generic_kernel(const T *x, T *y, size_t n) {
    for (size_t i = (size_t)blockIdx.x * kStreamThreads + threadIdx.x; i < n;
         i += (size_t)gridDim.x * kStreamThreads)
        Store<T>::store1(y + i, OP::apply(Store<T>::load1(x + i)));
}

// ===========================================================================
// Timestep embedding
// ===========================================================================
// freq_i is the float32 expression exp(neg_log_period * float(i) / float(half))
// with one rounding per operation; exp is evaluated in double and rounded once,
// which reproduces a correctly rounded float exp.  The angle float(t)*freq is a
// single float32 product; cos / sin are evaluated in double and rounded once.
template <typename T>
__global__ __launch_bounds__(256) void timestep_embedding_kernel(
    const int64_t *__restrict__ timesteps, T *__restrict__ out, uint32_t batch, uint32_t half,
    float neg_log_period) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= batch * half) return;
    const uint32_t b = idx / half, i = idx - b * half;
    const float z = __fdiv_rn(__fmul_rn(neg_log_period, (float)i), (float)half);
    const float freq = (float)exp((double)z);
    const float arg = __fmul_rn((float)timesteps[b], freq);
    double sn, cs;
    sincos((double)arg, &sn, &cs);
    T *row = out + (size_t)b * (2 * half);
    Store<T>::store1(row + i, (float)cs);
    Store<T>::store1(row + half + i, (float)sn);
}

// ===========================================================================
// Host side
// ===========================================================================
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

FastDiv make_fast_div(uint32_t d) {
    FastDiv fd{0u, 0u, d};
    if (d <= 1) return fd;
    uint32_t L = 0;
    while ((1ull << L) < d) L++;
    const unsigned long long num = 1ull << (31 + L);
    fd.mul = (uint32_t)((num + d - 1) / d);
    fd.shift = L - 1;
    return fd;
}

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

// Scratch is private to a (device, stream) pair: launches on one stream are
// ordered, so a unit's slots are never shared by two launches in flight.
hipError_t get_scratch(hipStream_t stream, GnScratch *out) {
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
    const size_t partial_bytes = sizeof(unsigned long long) * kGnMaxUnits * kGnMaxSplit;
    const size_t counter_bytes = sizeof(uint32_t) * kGnMaxUnits;
    char *base = nullptr;
    err = hipMalloc(reinterpret_cast<void **>(&base), partial_bytes + counter_bytes + 256);
    if (err != hipSuccess) return err;
    err = hipMemset(base, 0, partial_bytes + counter_bytes + 256);
    if (err != hipSuccess) {
        (void)hipFree(base);
        return err;
    }
    GnScratch s;
    s.partial = reinterpret_cast<unsigned long long *>(base);
    s.counter = reinterpret_cast<uint32_t *>(base + partial_bytes);
    s.status = reinterpret_cast<uint32_t *>(base + partial_bytes + counter_bytes);
    g_scratch.emplace(key, s);
    *out = s;
    return hipSuccess;
}

inline int launch_status() { return (int)hipGetLastError(); }

// ---- GroupNorm dispatch ----------------------------------------------------
uint32_t g_gn_target_blocks = 512;  // aim for about this many workgroups per launch

template <typename T, int K>
void gn_launch_k(bool silu, uint32_t blocks, hipStream_t stream, const T *x, T *y,
                 const float *gamma, const float *beta, const GnScratch &sc, const GnParams &p) {
    if (silu)
        hipLaunchKernelGGL((gn_split_kernel<T, K, true>), dim3(blocks), dim3(kGnThreads), 0, stream,
                           x, y, gamma, beta, sc, p);
    else
        hipLaunchKernelGGL((gn_split_kernel<T, K, false>), dim3(blocks), dim3(kGnThreads), 0,
                           stream, x, y, gamma, beta, sc, p);
}

template <typename T>
int gn_dispatch(const void *xv, void *yv, const float *gamma, const float *beta, size_t batch,
                size_t channels, size_t hw, size_t groups, float eps, bool silu,
                hipStream_t stream) {
    constexpr int EPV = Store<T>::EPV;
    constexpr uint32_t kMaxK = 8;
    const T *x = static_cast<const T *>(xv);
    T *y = static_cast<T *>(yv);
    const size_t cpg = channels / groups;
    const size_t unit_size = cpg * hw;
    const size_t units = batch * groups;
    if (units == 0 || unit_size == 0) return MSD_OK;
    if (units > 0x7FFFFFFFull || unit_size > 0x7FFFFFFFull) return MSD_ERR_INVALID_VALUE;

    const bool vector_ok = aligned16(x) && aligned16(y) && hw % EPV == 0;
    const size_t vec_per_unit = unit_size / EPV;
    // smallest power-of-two split that lets a slice fit K <= kMaxK vectors per lane
    uint32_t split = 1;
    while ((size_t)split * kGnThreads * kMaxK < vec_per_unit && split <= kGnMaxSplit) split *= 2;
    if (!vector_ok || split > kGnMaxSplit) {
        hipLaunchKernelGGL((silu ? gn_generic_kernel<T, true> : gn_generic_kernel<T, false>),
                           dim3((uint32_t)units), dim3(kGnThreads), 0, stream, x, y, gamma, beta,
                           (uint32_t)unit_size, (uint32_t)hw, (uint32_t)groups, (uint32_t)cpg, eps);
        return launch_status();
    }
    // widen the split for parallelism while every lane still has a vector
    if (units <= kGnMaxUnits)
        while (split < kGnMaxSplit && units * split < g_gn_target_blocks &&
               vec_per_unit >= (size_t)2 * split * kGnThreads)
            split *= 2;
    else if (split > 1) {
        hipLaunchKernelGGL((silu ? gn_generic_kernel<T, true> : gn_generic_kernel<T, false>),
                           dim3((uint32_t)units), dim3(kGnThreads), 0, stream, x, y, gamma, beta,
                           (uint32_t)unit_size, (uint32_t)hw, (uint32_t)groups, (uint32_t)cpg, eps);
        return launch_status();
    }

    GnParams p;
    p.vec_per_unit = (uint32_t)vec_per_unit;
    p.vec_per_slice = (uint32_t)((vec_per_unit + split - 1) / split);
    p.split = split;
    p.split_shift = (uint32_t)__builtin_ctz(split);
    p.groups = (uint32_t)groups;
    p.ch_per_group = (uint32_t)cpg;
    p.hw_vec = make_fast_div((uint32_t)(hw / EPV));
    p.eps = eps;
    p.inv_count = 1.0f / (float)unit_size;
    // ceil split can leave trailing slices empty; shrink so every slice owns a vector
    if ((size_t)p.vec_per_slice * (split - 1) >= vec_per_unit) {
        hipLaunchKernelGGL((silu ? gn_generic_kernel<T, true> : gn_generic_kernel<T, false>),
                           dim3((uint32_t)units), dim3(kGnThreads), 0, stream, x, y, gamma, beta,
                           (uint32_t)unit_size, (uint32_t)hw, (uint32_t)groups, (uint32_t)cpg, eps);
        return launch_status();
    }

    GnScratch sc{nullptr, nullptr, nullptr};
    if (split > 1) {
        const hipError_t err = get_scratch(stream, &sc);
        if (err != hipSuccess) return (int)err;
    }
    const uint32_t blocks = (uint32_t)(units * split);
    const uint32_t k = (p.vec_per_slice + kGnThreads - 1) / kGnThreads;
    switch (k) {
        case 1: gn_launch_k<T, 1>(silu, blocks, stream, x, y, gamma, beta, sc, p); break;
        case 2: gn_launch_k<T, 2>(silu, blocks, stream, x, y, gamma, beta, sc, p); break;
        case 3: gn_launch_k<T, 3>(silu, blocks, stream, x, y, gamma, beta, sc, p); break;
        case 4: gn_launch_k<T, 4>(silu, blocks, stream, x, y, gamma, beta, sc, p); break;
        case 5:
        case 6: gn_launch_k<T, 6>(silu, blocks, stream, x, y, gamma, beta, sc, p); break;
        default: gn_launch_k<T, 8>(silu, blocks, stream, x, y, gamma, beta, sc, p); break;
    }
    return launch_status();
}

// ---- LayerNorm dispatch ----------------------------------------------------
template <typename T, int VPL, int TL>
void ln_launch(const T *x, T *y, const float *gamma, const float *beta, uint32_t rows, float eps,
               float inv_dim, hipStream_t stream) {
    constexpr uint32_t rows_per_block = (kWave / TL) * (kLnThreads / kWave);
    const uint32_t blocks = (rows + rows_per_block - 1) / rows_per_block;
    hipLaunchKernelGGL((ln_team_kernel<T, VPL, TL>), dim3(blocks), dim3(kLnThreads), 0, stream, x, y,
                       gamma, beta, rows, eps, inv_dim);
}

template <typename T, int TL>
bool ln_launch_vpl(uint32_t vpl, const T *x, T *y, const float *gamma, const float *beta,
                   uint32_t rows, float eps, float inv_dim, hipStream_t stream) {
    switch (vpl) {
        case 1: ln_launch<T, 1, TL>(x, y, gamma, beta, rows, eps, inv_dim, stream); return true;
        case 2: ln_launch<T, 2, TL>(x, y, gamma, beta, rows, eps, inv_dim, stream); return true;
        case 3: ln_launch<T, 3, TL>(x, y, gamma, beta, rows, eps, inv_dim, stream); return true;
        case 4: ln_launch<T, 4, TL>(x, y, gamma, beta, rows, eps, inv_dim, stream); return true;
        case 5: ln_launch<T, 5, TL>(x, y, gamma, beta, rows, eps, inv_dim, stream); return true;
        case 6: ln_launch<T, 6, TL>(x, y, gamma, beta, rows, eps, inv_dim, stream); return true;
        case 7: ln_launch<T, 7, TL>(x, y, gamma, beta, rows, eps, inv_dim, stream); return true;
        case 8: ln_launch<T, 8, TL>(x, y, gamma, beta, rows, eps, inv_dim, stream); return true;
        default: return false;
    }
}

template <typename T>
int ln_dispatch(const void *xv, void *yv, const float *gamma, const float *beta, size_t rows,
                size_t dim, float eps, hipStream_t stream) {
    constexpr int EPV = Store<T>::EPV;
    const T *x = static_cast<const T *>(xv);
    T *y = static_cast<T *>(yv);
    if (rows == 0 || dim == 0) return MSD_OK;
    if (rows > 0x7FFFFFFFull || dim > 0x7FFFFFFFull) return MSD_ERR_INVALID_VALUE;
    const float inv_dim = 1.0f / (float)dim;
    bool done = false;
    if (aligned16(x) && aligned16(y) && aligned16(gamma) && aligned16(beta) && dim % EPV == 0) {
        const uint32_t vec_per_row = (uint32_t)(dim / EPV);
        uint32_t tl = kWave;
        while (vec_per_row % tl != 0) tl /= 2;
        const uint32_t vpl = vec_per_row / tl;
        const uint32_t r = (uint32_t)rows;
        switch (tl) {
            case 64: done = ln_launch_vpl<T, 64>(vpl, x, y, gamma, beta, r, eps, inv_dim, stream); break;
            case 32: done = ln_launch_vpl<T, 32>(vpl, x, y, gamma, beta, r, eps, inv_dim, stream); break;
            case 16: done = ln_launch_vpl<T, 16>(vpl, x, y, gamma, beta, r, eps, inv_dim, stream); break;
            case 8: done = ln_launch_vpl<T, 8>(vpl, x, y, gamma, beta, r, eps, inv_dim, stream); break;
            case 4: done = ln_launch_vpl<T, 4>(vpl, x, y, gamma, beta, r, eps, inv_dim, stream); break;
            default: break;
        }
    }
    if (!done) {
        const uint32_t rows_per_block = kLnThreads / kWave;
        hipLaunchKernelGGL((ln_generic_kernel<T>),
                           dim3((uint32_t)((rows + rows_per_block - 1) / rows_per_block)),
                           dim3(kLnThreads), 0, stream, x, y, gamma, beta, (uint32_t)rows,
                           (uint32_t)dim, eps);
    }
    return launch_status();
}

// ---- streaming dispatch ----------------------------------------------------
inline uint32_t stream_blocks(size_t vecs) {
    const size_t per_block = (size_t)kStreamThreads * kStreamUnroll;
    return (uint32_t)((vecs + per_block - 1) / per_block);
}

template <typename T>
int geglu_dispatch(const void *pv, void *ov, size_t rows, size_t inner, hipStream_t stream) {
    constexpr int EPV = Store<T>::EPV;
    const T *proj = static_cast<const T *>(pv);
    T *out = static_cast<T *>(ov);
    if (rows == 0 || inner == 0) return MSD_OK;
    const size_t out_vecs = rows * (inner / EPV);
    if (aligned16(proj) && aligned16(out) && inner % EPV == 0 && out_vecs < 0x7FFFFFFFull &&
        rows < 0x7FFFFFFFull) {
        hipLaunchKernelGGL((geglu_kernel<T>), dim3(stream_blocks(out_vecs)), dim3(kStreamThreads),
                           0, stream, proj, out, (uint32_t)out_vecs,
                           make_fast_div((uint32_t)(inner / EPV)));
    } else {
        const size_t n = rows * inner;
        const size_t want = (n + kStreamThreads - 1) / kStreamThreads;
        hipLaunchKernelGGL((geglu_generic_kernel<T>), dim3((uint32_t)(want < 65536 ? want : 65536)),
                           dim3(kStreamThreads), 0, stream, proj, out, rows, inner);
    }
    return launch_status();
}

template <typename T, typename OP>
int act_dispatch(const void *xv, void *yv, size_t n, hipStream_t stream) {
    constexpr int EPV = Store<T>::EPV;
    const T *x = static_cast<const T *>(xv);
    T *y = static_cast<T *>(yv);
    if (n == 0) return MSD_OK;
    const size_t vecs = n / EPV;
    if (aligned16(x) && aligned16(y) && vecs < 0x7FFFFFFFull) {
        const uint32_t blocks = vecs ? stream_blocks(vecs) : 1u;
        hipLaunchKernelGGL((act_kernel<T, OP>), dim3(blocks), dim3(kStreamThreads), 0, stream, x, y,
                           (uint32_t)vecs, n);
    } else {
        const size_t want = (n + kStreamThreads - 1) / kStreamThreads;
        hipLaunchKernelGGL((act_generic_kernel<T, OP>),
                           dim3((uint32_t)(want < 65536 ? want : 65536)), dim3(kStreamThreads), 0,
                           stream, x, y, n);
    }
    return launch_status();
}

template <typename OP>
int act_entry(const void *x, void *y, size_t n, int dtype, void *stream) {
    if ((!x || !y) && n != 0) return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MSD_DTYPE_F32) return act_dispatch<float, OP>(x, y, n, s);
    if (dtype == MSD_DTYPE_F16) return act_dispatch<__half, OP>(x, y, n, s);
    return MSD_ERR_INVALID_VALUE;
}

}  // namespace

// ===========================================================================
// C ABI
// ===========================================================================
extern "C" {

int msd_version(void) { return 100; }

const char *msd_error_string(int code) {
    if (code == MSD_OK) return "ok";
    if (code == MSD_ERR_INVALID_VALUE) return "invalid value (shape, pointer or dtype rejected)";
    return hipGetErrorString(static_cast<hipError_t>(code));
}

int msd_init(void *stream) {
    GnScratch sc;
    return (int)get_scratch(static_cast<hipStream_t>(stream), &sc);
}

int msd_shutdown(void) {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    int rc = MSD_OK;
    int current = 0;
    (void)hipGetDevice(&current);
    for (auto &kv : g_scratch) {
        (void)hipSetDevice(kv.first.device);
        const hipError_t err = hipFree(kv.second.partial);
        if (err != hipSuccess) rc = (int)err;
    }
    g_scratch.clear();
    (void)hipSetDevice(current);
    return rc;
}

int msd_status(void *stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t err = hipStreamSynchronize(s);
    if (err != hipSuccess) return (int)err;
    int device = 0;
    err = hipGetDevice(&device);
    if (err != hipSuccess) return (int)err;
    GnScratch sc{nullptr, nullptr, nullptr};
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        auto it = g_scratch.find(ScratchKey{device, s});
        if (it == g_scratch.end()) return MSD_OK;
        sc = it->second;
    }
    uint32_t flags = 0;
    err = hipMemcpy(&flags, sc.status, sizeof(flags), hipMemcpyDeviceToHost);
    if (err != hipSuccess) return (int)err;
    return flags ? (int)hipErrorLaunchFailure : MSD_OK;
}

int msd_set_groupnorm_target_blocks(int blocks) {
    if (blocks < 1) return MSD_ERR_INVALID_VALUE;
    g_gn_target_blocks = (uint32_t)blocks;
    return MSD_OK;
}

int msd_groupnorm(const void *x, void *y, const float *gamma, const float *beta, size_t batch,
                  size_t channels, size_t hw, size_t groups, float eps, int fuse_silu, int dtype,
                  void *stream) {
    if (groups == 0 || channels == 0 || channels % groups != 0) return MSD_ERR_INVALID_VALUE;
    if (batch * hw != 0 && (!x || !y || !gamma || !beta)) return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MSD_DTYPE_F32)
        return gn_dispatch<float>(x, y, gamma, beta, batch, channels, hw, groups, eps,
                                  fuse_silu != 0, s);
    if (dtype == MSD_DTYPE_F16)
        return gn_dispatch<__half>(x, y, gamma, beta, batch, channels, hw, groups, eps,
                                   fuse_silu != 0, s);
    return MSD_ERR_INVALID_VALUE;
}

int msd_layernorm(const void *x, void *y, const float *gamma, const float *beta, size_t rows,
                  size_t dim, float eps, int dtype, void *stream) {
    if (rows * dim != 0 && (!x || !y || !gamma || !beta)) return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MSD_DTYPE_F32) return ln_dispatch<float>(x, y, gamma, beta, rows, dim, eps, s);
    if (dtype == MSD_DTYPE_F16) return ln_dispatch<__half>(x, y, gamma, beta, rows, dim, eps, s);
    return MSD_ERR_INVALID_VALUE;
}

int msd_geglu(const void *proj, void *out, size_t rows, size_t inner, int dtype, void *stream) {
    if (rows * inner != 0 && (!proj || !out)) return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MSD_DTYPE_F32) return geglu_dispatch<float>(proj, out, rows, inner, s);
    if (dtype == MSD_DTYPE_F16) return geglu_dispatch<__half>(proj, out, rows, inner, s);
    return MSD_ERR_INVALID_VALUE;
}

int msd_silu(const void *x, void *y, size_t n, int dtype, void *stream) {
    return act_entry<OpSilu>(x, y, n, dtype, stream);
}
int msd_gelu(const void *x, void *y, size_t n, int dtype, void *stream) {
    return act_entry<OpGelu>(x, y, n, dtype, stream);
}
int msd_quick_gelu(const void *x, void *y, size_t n, int dtype, void *stream) {
    return act_entry<OpQuickGelu>(x, y, n, dtype, stream);
}

int msd_timestep_embedding(const int64_t *timesteps, void *out, size_t batch, size_t dim,
                           float max_period, int dtype, void *stream) {
    if (dim % 2 != 0 || !(max_period > 0.0f)) return MSD_ERR_INVALID_VALUE;
    if (batch * dim == 0) return MSD_OK;
    if (!timesteps || !out || batch * dim > 0x7FFFFFFFull) return MSD_ERR_INVALID_VALUE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint32_t half = (uint32_t)(dim / 2);
    const uint32_t blocks = (uint32_t)((batch * half + 255) / 256);
    const float neg_log_period = -logf(max_period);  // host float log, as the replaced host loop
    if (dtype == MSD_DTYPE_F32)
        hipLaunchKernelGGL((timestep_embedding_kernel<float>), dim3(blocks), dim3(256), 0, s,
                           timesteps, static_cast<float *>(out), (uint32_t)batch, half,
                           neg_log_period);
    else if (dtype == MSD_DTYPE_F16)
        hipLaunchKernelGGL((timestep_embedding_kernel<__half>), dim3(blocks), dim3(256), 0, s,
                           timesteps, static_cast<__half *>(out), (uint32_t)batch, half,
                           neg_log_period);
    else
        return MSD_ERR_INVALID_VALUE;
    return launch_status();
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

}  // extern "C"
