// LayerNorm for gfx950: a row is owned by a team of TL adjacent lanes of one
// wavefront (TL = 4..64), VPL 16-byte vectors per lane, so a wavefront covers
// 64/TL consecutive rows and every load instruction fetches whole 128-byte lines.
// Mean and M2 come from one pass of sum and sum of squares over the packed registers, reduced
// across the team with DPP; a wavefront in which some row's mean is large against its spread
// (|mean| > 2 sigma, or a constant row) takes a second, centred pass over the registers, so the
// variance is as accurate as a two-pass one either way.  gamma / beta are fetched while the row
// data is in flight (small launches) or staged in LDS once per workgroup.  One HBM read and one
// HBM write per element.
#include "msd_device.h"
#include "msd_internal.h"

namespace msd {
namespace {

constexpr int kLnThreads = 64;      // workgroup of the scalar kernel; smallest team-kernel workgroup
constexpr int kLnMaxThreads = 512;  // launch bound

// NW dwords (8 or 16 bytes) of T, moved with one instruction.
template <int NW>
struct Words;
template <>
struct Words<4> {
    typedef u32x4 type;
};
template <>
struct Words<2> {
    typedef uint32_t type __attribute__((ext_vector_type(2)));
};

template <typename T, int NW>
struct Chunk {
    static constexpr int N = NW * 4 / (int)sizeof(T);  // elements per chunk
    typedef typename Words<NW>::type vec_t;
    static __device__ __forceinline__ void unpack(const vec_t &v, float *f) {
        if (sizeof(T) == 4) {
#pragma unroll
            for (int i = 0; i < NW; i++) f[i] = __uint_as_float(v[i]);
        } else {
#pragma unroll
            for (int i = 0; i < NW; i++) {
                const uint32_t w = v[i];
                const float2 t = __half22float2(*reinterpret_cast<const __half2 *>(&w));
                f[2 * i] = t.x;
                f[2 * i + 1] = t.y;
            }
        }
    }
    static __device__ __forceinline__ vec_t pack(const float *f) {
        vec_t v;
        if (sizeof(T) == 4) {
#pragma unroll
            for (int i = 0; i < NW; i++) v[i] = __float_as_uint(f[i]);
        } else {
#pragma unroll
            for (int i = 0; i < NW; i++) {
                const __half2 h = __floats2half2_rn(f[2 * i], f[2 * i + 1]);
                v[i] = *reinterpret_cast<const uint32_t *>(&h);
            }
        }
        return v;
    }
};

// Sum and sum of squares of the packed words of a chunk, accumulated in float32 (half storage:
// v_dot2_f32_f16, whose two products are exact in float32; subnormal halves count).
template <typename T, int NW>
__device__ __forceinline__ void chunk_moments(const typename Words<NW>::type &v, float (&s)[2], float (&q)[2]) {
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int i = 0; i < NW; i++) {
        if (sizeof(T) == 4) {
            const float f = __uint_as_float(v[i]);
            s[i & 1] += f;
            q[i & 1] = fmaf(f, f, q[i & 1]);
        } else {
            const half2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
            const uint32_t w = v[i];
            const half2_t h = *reinterpret_cast<const half2_t *>(&w);
            s[i & 1] = __builtin_amdgcn_fdot2(h, ones, s[i & 1], false);
            q[i & 1] = __builtin_amdgcn_fdot2(h, h, q[i & 1], false);
        }
    }
}

// |mean| <= 2 sigma: a row's M2 may be taken from its raw moments (relative error below 1e-6)
constexpr float kLnFastMoments = 4.0f;

// A row of VPL*TL chunks (NW dwords each) is owned by TL adjacent lanes; a wavefront
// covers 64/TL consecutive rows.  Lane (team, j) holds chunks j, j+TL, ... of its row, all
// requested before the first use.  One pass over the packed registers gives the row's sum and
// sum of squares (team reduction by DPP); M2 = sum x^2 - n mean^2 is kept when it is well
// conditioned, otherwise (a wavefront-uniform branch taken when any of its rows needs it) a
// second pass sums (x - mean)^2.  The epilogue unpacks one chunk at a time, so the row never
// sits in registers twice.  gamma / beta of the lane's columns are requested together with
// the row when EARLY (short launches: one memory latency instead of two on the critical path,
// at the price of 2 * VPL * N registers).  Otherwise (long launches, bound by throughput) the
// workgroup copies gamma and beta into LDS once while its rows are in flight and every lane
// reads its columns from there: fetching them from the cache per row costs four times the
// row's own bytes in load instructions (measured at 131072 x 320 fp16: 31.2 us from global
// memory, 29.7 us from LDS, 29.4 us with no affine at all).
template <typename T, int NW, int VPL, int TL, bool EARLY>
__global__ __launch_bounds__(kLnMaxThreads) void ln_team_kernel(
    const T *x, const T *res, T *sum, T *y, const float *__restrict__ gamma,
    const float *__restrict__ beta, uint32_t rows, float eps, float inv_dim) {
    typedef Chunk<T, NW> C;
    typedef typename C::vec_t vec_t;
    constexpr int N = C::N;
    constexpr int RPW = kWave / TL;  // rows per wavefront
    constexpr int DIM = VPL * TL * N;
    extern __shared__ f32x4 ln_lds[];  // !EARLY: gamma[DIM] then beta[DIM]
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
    const uint32_t row = wave * RPW + lane / TL;
    const uint32_t j = lane % TL;
    const bool live = row < rows;
    // lanes past the last row re-read it (valid address, no branch around the loads)
    const size_t row_chunk = (size_t)min(row, rows - 1) * (VPL * TL);
    const vec_t *xin = reinterpret_cast<const vec_t *>(x) + row_chunk;
    vec_t *yout = reinterpret_cast<vec_t *>(y) + row_chunk;

    vec_t raw[VPL];
#pragma unroll
    for (int k = 0; k < VPL; k++) raw[k] = __builtin_nontemporal_load(xin + k * TL + j);
    if (res != nullptr) {  // uniform: residual to add before the norm (the reference's elemwise_add)
        const vec_t *rin = reinterpret_cast<const vec_t *>(res) + row_chunk;
        vec_t *sout = reinterpret_cast<vec_t *>(sum) + row_chunk;
        vec_t raw_res[VPL];
#pragma unroll
        for (int k = 0; k < VPL; k++) raw_res[k] = __builtin_nontemporal_load(rin + k * TL + j);
        // x + res, rounded to the storage type and written out exactly as a separate add kernel
        // would have left it; the norm then works on those stored values
#pragma unroll
        for (int k = 0; k < VPL; k++) {
            float f[N], r[N];
            C::unpack(raw[k], f);
            C::unpack(raw_res[k], r);
#pragma unroll
            for (int e = 0; e < N; e++) f[e] += r[e];
            raw[k] = C::pack(f);
            if (live) __builtin_nontemporal_store(raw[k], sout + k * TL + j);
        }
    }
    if (!EARLY) {  // the whole workgroup, rows past the end included, fills the LDS copy
        for (uint32_t i = threadIdx.x; i < DIM / 4; i += blockDim.x) {
            ln_lds[i] = reinterpret_cast<const f32x4 *>(gamma)[i];
            ln_lds[DIM / 4 + i] = reinterpret_cast<const f32x4 *>(beta)[i];
        }
    }
    // gamma / beta of chunk k's columns, from global memory or from the LDS copy
    auto affine = [&](const float *gsrc, const float *bsrc, int k, float (&g)[N], float (&b)[N]) {
        const uint32_t col = (k * TL + j) * N;
#pragma unroll
        for (int e = 0; e < N; e += (N >= 4 ? 4 : 2)) {
            if (N >= 4) {
                const f32x4 gv = *reinterpret_cast<const f32x4 *>(gsrc + col + e);
                const f32x4 bv = *reinterpret_cast<const f32x4 *>(bsrc + col + e);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    g[e + i] = gv[i];
                    b[e + i] = bv[i];
                }
            } else {
                const float2 gv = *reinterpret_cast<const float2 *>(gsrc + col + e);
                const float2 bv = *reinterpret_cast<const float2 *>(bsrc + col + e);
                g[e] = gv.x;
                g[e + 1] = gv.y;
                b[e] = bv.x;
                b[e + 1] = bv.y;
            }
        }
    };
    float g_all[EARLY ? VPL : 1][N], b_all[EARLY ? VPL : 1][N];
    if (EARLY) {
#pragma unroll
        for (int k = 0; k < VPL; k++) affine(gamma, beta, k, g_all[EARLY ? k : 0], b_all[EARLY ? k : 0]);
    }
    float s[2] = {0.0f, 0.0f}, q[2] = {0.0f, 0.0f};
#pragma unroll
    for (int k = 0; k < VPL; k++) chunk_moments<T, NW>(raw[k], s, q);
    const float sum_x = team_sum<TL>(s[0] + s[1]);
    const float sum_xx = team_sum<TL>(q[0] + q[1]);
    const float mean = sum_x * inv_dim;
    float m2 = sum_xx - sum_x * mean;
    const bool fast = sum_x * mean <= kLnFastMoments * m2;  // false also for a negative or NaN M2
    if (__builtin_amdgcn_ballot_w64(!fast) != 0) {  // some row of this wavefront needs the exact M2
        float c = 0.0f;
#pragma unroll
        for (int k = 0; k < VPL; k++) {
            float f[N];
            C::unpack(raw[k], f);
#pragma unroll
            for (int e = 0; e < N; e++) {
                const float d = f[e] - mean;
                c = fmaf(d, d, c);
            }
        }
        const float exact = team_sum<TL>(c);
        m2 = fast ? m2 : exact;
    }
    const float rstd = __builtin_amdgcn_rsqf(m2 * inv_dim + eps);
    if (!EARLY) __syncthreads();  // the LDS copy of gamma / beta is complete
    if (!live) return;
#pragma unroll
    for (int k = 0; k < VPL; k++) {
        float g[N], b[N];
        if (EARLY) {
#pragma unroll
            for (int e = 0; e < N; e++) {
                g[e] = g_all[EARLY ? k : 0][e];
                b[e] = b_all[EARLY ? k : 0][e];
            }
        } else {
            affine(reinterpret_cast<const float *>(ln_lds), reinterpret_cast<const float *>(ln_lds) + DIM, k, g, b);
        }
        float f[N], o[N];
        C::unpack(raw[k], f);
#pragma unroll
        for (int e = 0; e < N; e++) o[e] = fmaf((f[e] - mean) * rstd, g[e], b[e]);
        __builtin_nontemporal_store(C::pack(o), yout + k * TL + j);
    }
}

// Any dim: one wavefront per row, scalar accesses, three passes.
template <typename T>
__global__ __launch_bounds__(kLnThreads) void ln_generic_kernel(
    const T *x, const T *res, T *sum, T *y, const float *__restrict__ gamma,
    const float *__restrict__ beta, uint32_t rows, uint32_t dim, float eps) {
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t row = blockIdx.x * (kLnThreads / kWave) + threadIdx.x / kWave;
    if (row >= rows) return;  // whole wavefront leaves together
    const T *xin = x + (size_t)row * dim;
    T *yout = y + (size_t)row * dim;
    if (res != nullptr) {  // write x + res first; each lane later re-reads only what it wrote
        const T *rin = res + (size_t)row * dim;
        T *sout = sum + (size_t)row * dim;
        for (uint32_t i = lane; i < dim; i += kWave)
            Store<T>::store1(sout + i, Store<T>::load1(xin + i) + Store<T>::load1(rin + i));
        xin = sout;
    }
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

// ---- LayerNorm dispatch ----------------------------------------------------
template <typename T, int NW, int VPL, int TL>
void ln_launch(const T *x, const T *res, T *sum, T *y, const float *gamma, const float *beta,
               uint32_t rows, float eps, float inv_dim, hipStream_t stream) {
    // Up to one wavefront per SIMD of the chip (four SIMDs per CU) the launch is bound by its own latency chain:
    // one wavefront per workgroup (1 - 5 % faster than four), gamma / beta requested together with
    // the row.  From two wavefronts per SIMD on throughput counts: gamma / beta through LDS (fewer
    // load instructions and registers per wavefront), four wavefronts per workgroup, two for
    // launches of four up to ten wavefronts per SIMD (3 - 19 % faster there, 1 - 7 % slower at three
    // and from ten on).  Measured, us per launch, with the row / LDS x 64, 128, 256 lanes:
    //   fp16 8192 x 320 (1024 wavefronts)   3.54 3.71 3.59 / 3.57 3.88 3.57
    //   fp16 16384 x 320 (2048)             5.12 5.19 5.22 / 4.94 4.78 4.94
    //   fp32 8192 x 320 (2048)              5.28 5.29 5.17 / 4.90 4.71 4.99
    //   fp16 8192 x 1024 (8192)             8.19 8.01 8.17 / 9.32 7.09 7.96
    //   fp16 16384 x 768 (8192)             11.8 12.1 12.2 / 12.1 9.54 10.7
    //   fp16 8192 x 1280 (4096)             10.4 10.6 10.4 / 8.19 7.95 7.95
    //   fp16 32768 x 1024 (32768)           24.5 24.5 24.5 / 31.7 25.0 24.1
    const uint32_t wavefronts = (rows + (kWave / TL) - 1) / (kWave / TL);
    const uint32_t simds = 4 * chip_info().cus;  // (the figures above: 1024 SIMDs)
    const bool early = wavefronts < 2 * simds;
    const int tune_threads = g_tuning.ln_threads.load(std::memory_order_relaxed);
    const uint32_t threads = tune_threads ? (uint32_t)tune_threads
                             : early      ? (wavefronts <= simds ? (uint32_t)kLnThreads : 256u)
                                          : (wavefronts >= 4 * simds && wavefronts < 10 * simds ? 128u : 256u);
    const uint32_t rows_per_block = (kWave / TL) * (threads / kWave);
    const uint32_t blocks = (rows + rows_per_block - 1) / rows_per_block;
    if (early)
        launch((ln_team_kernel<T, NW, VPL, TL, true>), dim3(blocks), dim3(threads), 0, stream, x,
                           res, sum, y, gamma, beta, rows, eps, inv_dim);
    else
        launch((ln_team_kernel<T, NW, VPL, TL, false>), dim3(blocks), dim3(threads),
                           2 * sizeof(float) * VPL * TL * (NW * 4 / sizeof(T)), stream, x, res, sum, y, gamma, beta,
                           rows, eps, inv_dim);
}

template <typename T, int NW, int TL>
bool ln_launch_vpl(uint32_t vpl, const T *x, const T *res, T *sum, T *y, const float *gamma,
                   const float *beta, uint32_t rows, float eps, float inv_dim, hipStream_t stream) {
    switch (vpl) {
        case 1: ln_launch<T, NW, 1, TL>(x, res, sum, y, gamma, beta, rows, eps, inv_dim, stream); return true;
        case 2: ln_launch<T, NW, 2, TL>(x, res, sum, y, gamma, beta, rows, eps, inv_dim, stream); return true;
        case 3: ln_launch<T, NW, 3, TL>(x, res, sum, y, gamma, beta, rows, eps, inv_dim, stream); return true;
        case 4: ln_launch<T, NW, 4, TL>(x, res, sum, y, gamma, beta, rows, eps, inv_dim, stream); return true;
        case 5: ln_launch<T, NW, 5, TL>(x, res, sum, y, gamma, beta, rows, eps, inv_dim, stream); return true;
        case 6: ln_launch<T, NW, 6, TL>(x, res, sum, y, gamma, beta, rows, eps, inv_dim, stream); return true;
        case 7: ln_launch<T, NW, 7, TL>(x, res, sum, y, gamma, beta, rows, eps, inv_dim, stream); return true;
        case 8: ln_launch<T, NW, 8, TL>(x, res, sum, y, gamma, beta, rows, eps, inv_dim, stream); return true;
        default: return false;
    }
}

// Tries the team kernel with NW-dword chunks; false when the row does not decompose.
template <typename T, int NW>
bool ln_try(const T *x, const T *res, T *sum, T *y, const float *gamma, const float *beta,
            uint32_t rows, uint32_t dim, float eps, float inv_dim, hipStream_t stream) {
    constexpr uint32_t N = NW * 4 / sizeof(T);
    if (dim % N != 0) return false;
    const uint32_t chunks = dim / N;
    uint32_t tl = kWave;
    while (chunks % tl != 0) tl /= 2;
    const uint32_t vpl = chunks / tl;
    switch (tl) {
        case 64: return ln_launch_vpl<T, NW, 64>(vpl, x, res, sum, y, gamma, beta, rows, eps, inv_dim, stream);
        case 32: return ln_launch_vpl<T, NW, 32>(vpl, x, res, sum, y, gamma, beta, rows, eps, inv_dim, stream);
        case 16: return ln_launch_vpl<T, NW, 16>(vpl, x, res, sum, y, gamma, beta, rows, eps, inv_dim, stream);
        case 8: return ln_launch_vpl<T, NW, 8>(vpl, x, res, sum, y, gamma, beta, rows, eps, inv_dim, stream);
        case 4: return ln_launch_vpl<T, NW, 4>(vpl, x, res, sum, y, gamma, beta, rows, eps, inv_dim, stream);
        default: return false;
    }
}

}  // namespace

template <typename T>
int ln_dispatch(const void *xv, const void *resv, void *sumv, void *yv, const float *gamma,
                const float *beta, size_t rows, size_t dim, float eps, hipStream_t stream) {
    const T *x = static_cast<const T *>(xv);
    const T *res = static_cast<const T *>(resv);
    T *sum = static_cast<T *>(sumv);
    T *y = static_cast<T *>(yv);
    if (rows == 0 || dim == 0) return MSD_OK;
    if (rows > 0x7FFFFFFFull || dim > 0x7FFFFFFFull) return MSD_ERR_INVALID_VALUE;
    const float inv_dim = 1.0f / (float)dim;
    const uint32_t r = (uint32_t)rows, d = (uint32_t)dim;
    bool done = false;
    if (aligned16(x) && aligned16(y) && aligned16(gamma) && aligned16(beta) &&
        (res == nullptr || (aligned16(res) && aligned16(sum)))) {
        // A lane's dependent chain (convert, two reductions, affine) is on the critical path
        // of a launch this short, so half-precision rows are spread over more lanes with
        // 8-byte chunks when 16-byte ones would leave a team of fewer than 64 lanes with more
        // than 16 elements per lane (measured 10-20 % faster at dim 320 / 640 / 1280); float
        // rows keep 16-byte chunks (8-byte ones only add load instructions).
        const uint32_t n16 = 16 / sizeof(T);
        bool prefer8 = false;
        if (sizeof(T) == 2 && d % n16 == 0) {
            uint32_t tl = kWave;
            while ((d / n16) % tl != 0) tl /= 2;
            prefer8 = tl < kWave && (d / tl) > 16;
            // ... unless 16-byte chunks still give every SIMD of the chip a wavefront: then the
            // wider accesses win (8192 x 320: 3.7 against 3.9 us, with the residual 5.0 against 5.8)
            const size_t waves16 = (rows + kWave / tl - 1) / (kWave / tl);
            if (waves16 >= 1024) prefer8 = false;
        }
        const int tune_chunk = g_tuning.ln_chunk.load(std::memory_order_relaxed);
        if (tune_chunk == 8) prefer8 = true;
        if (tune_chunk == 16) prefer8 = false;
        if (prefer8) done = ln_try<T, 2>(x, res, sum, y, gamma, beta, r, d, eps, inv_dim, stream);
        if (!done) done = ln_try<T, 4>(x, res, sum, y, gamma, beta, r, d, eps, inv_dim, stream);
        if (!done && !prefer8) done = ln_try<T, 2>(x, res, sum, y, gamma, beta, r, d, eps, inv_dim, stream);
    }
    if (!done) {
        const uint32_t rows_per_block = kLnThreads / kWave;
        launch((ln_generic_kernel<T>),
                           dim3((uint32_t)((rows + rows_per_block - 1) / rows_per_block)),
                           dim3(kLnThreads), 0, stream, x, res, sum, y, gamma, beta, (uint32_t)rows,
                           (uint32_t)dim, eps);
    }
    return launch_status();
}

template int ln_dispatch<float>(const void *, const void *, void *, void *, const float *,
                                const float *, size_t, size_t, float, hipStream_t);
template int ln_dispatch<__half>(const void *, const void *, void *, void *, const float *,
                                 const float *, size_t, size_t, float, hipStream_t);

}  // namespace msd
