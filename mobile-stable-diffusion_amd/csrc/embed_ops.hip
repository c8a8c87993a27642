// Neighbours of the norm / activation path for gfx950: the Linear layers that act on
// the few rows of the time embedding (weight-streaming, one output column per
// wavefront), the row softmax of the attention blocks (a row held in the registers
// of a team of lanes) and the DDIM latent update.
#include "msd_device.h"
#include "msd_internal.h"

#include <cmath>

namespace msd {
namespace {

// ---------------------------------------------------------------------------
// y[m, n] = act_out(act_in(x)[m, k] . w[n, k]^T + bias[n]) for m <= 8 rows.
// The time is the single pass over w (n*k elements); x is staged once per workgroup
// in LDS as float with act_in already applied.  A wavefront owns one column: lane l
// multiplies 16-byte pieces l, l+64, ... of the weight row, every load of a round of
// UN pieces issued before the first use, then the M partial sums go through the DPP
// tree.  Each lane adds its pieces in ascending k; the tree order is fixed, so the
// result does not depend on the launch shape.
// ---------------------------------------------------------------------------
constexpr int kLinThreads = 256;
constexpr int kLinWaves = kLinThreads / kWave;
constexpr int kLinRound = 4;            // 16-byte weight loads in flight per lane
constexpr size_t kLinMaxStaged = 12288; // floats of x in LDS (48 KiB)

template <typename T, int M>
__global__ __launch_bounds__(kLinThreads) void linear_rows_kernel(
    const T *__restrict__ x, const T *__restrict__ w, const float *__restrict__ bias,
    T *__restrict__ y, uint32_t m, uint32_t n, uint32_t kvecs, int act_in, int act_out) {
    constexpr int EPV = Store<T>::EPV;
    extern __shared__ float xs[];  // [M][kvecs * EPV]
    const uint32_t k = kvecs * EPV;
    const u32x4 *xin = reinterpret_cast<const u32x4 *>(x);
    for (uint32_t v = threadIdx.x; v < M * kvecs; v += kLinThreads) {
        const uint32_t row = v / kvecs, piece = v - row * kvecs;
        float f[EPV];
        Store<T>::unpack(xin[(size_t)min(row, m - 1) * kvecs + piece], f);  // rows >= m repeat the last
        if (act_in) {
#pragma unroll
            for (int e = 0; e < EPV; e++) f[e] = silu_f(f[e]);
        }
#pragma unroll
        for (int e = 0; e < EPV; e++) xs[row * k + piece * EPV + e] = f[e];
    }
    __syncthreads();
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t col = blockIdx.x * kLinWaves + threadIdx.x / kWave;
    if (col >= n) return;  // whole wavefront; no barrier follows
    const u32x4 *wrow = reinterpret_cast<const u32x4 *>(w) + (size_t)col * kvecs;
    float acc[M];
#pragma unroll
    for (int i = 0; i < M; i++) acc[i] = 0.0f;
    for (uint32_t base = lane; base < kvecs; base += kWave * kLinRound) {
        u32x4 raw[kLinRound];
#pragma unroll
        for (int u = 0; u < kLinRound; u++)
            raw[u] = load_stream(wrow + min(base + u * kWave, kvecs - 1));
#pragma unroll
        for (int u = 0; u < kLinRound; u++) {
            const uint32_t piece = base + u * kWave;
            if (piece < kvecs) {
                float wf[EPV];
                Store<T>::unpack(raw[u], wf);
#pragma unroll
                for (int i = 0; i < M; i++) {
                    const float *xr = xs + i * k + piece * EPV;
#pragma unroll
                    for (int e = 0; e < EPV; e++) acc[i] = fmaf(xr[e], wf[e], acc[i]);
                }
            }
        }
    }
    float mine = 0.0f;
#pragma unroll
    for (int i = 0; i < M; i++) {
        const float total = wave_sum(acc[i]);
        if (lane == (uint32_t)i) mine = total;
    }
    if (lane < m) {
        float r = mine + (bias != nullptr ? bias[col] : 0.0f);
        if (act_out) r = silu_f(r);
        Store<T>::store1(y + (size_t)lane * n + col, r);
    }
}

// Any k / alignment: x is read from global memory (it is a few KiB and stays cached).
template <typename T>
__global__ __launch_bounds__(kLinThreads) void linear_rows_generic_kernel(
    const T *__restrict__ x, const T *__restrict__ w, const float *__restrict__ bias,
    T *__restrict__ y, uint32_t m, uint32_t n, uint32_t k, int act_in, int act_out) {
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t col = blockIdx.x * kLinWaves + threadIdx.x / kWave;
    if (col >= n) return;
    const T *wrow = w + (size_t)col * k;
    for (uint32_t i = 0; i < m; i++) {
        float acc = 0.0f;
        for (uint32_t kk = lane; kk < k; kk += kWave) {
            float xv = Store<T>::load1(x + (size_t)i * k + kk);
            if (act_in) xv = silu_f(xv);
            acc = fmaf(xv, Store<T>::load1(wrow + kk), acc);
        }
        acc = wave_sum(acc);
        if (lane == 0) {
            float r = acc + (bias != nullptr ? bias[col] : 0.0f);
            if (act_out) r = silu_f(r);
            Store<T>::store1(y + (size_t)i * n + col, r);
        }
    }
}

// ---------------------------------------------------------------------------
// Row softmax.  exp(x - shift) / sum, shift = the row maximum (stable) or 0 (the
// form the replaced kernel computes, which overflows above x = 88.7 exactly as it
// does).  A row lives in the registers of a team of TL lanes, VPL 16-byte vectors
// per lane: one read and one write per element.  exp goes through the hardware 2^x
// (relative error below 1.2e-7 * (1 + |x - shift| * 1.45)).
// ---------------------------------------------------------------------------
constexpr int kSmThreads = 256;
constexpr float kNegInf = -__builtin_huge_valf();

template <typename T, int VPL, int TL>
__global__ __launch_bounds__(kSmThreads) void softmax_team_kernel(const T *x, T *y, uint32_t rows,
                                                                  uint32_t row_vecs, int stable) {
    constexpr int EPV = Store<T>::EPV;
    constexpr int RPW = kWave / TL;
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = blockIdx.x * (kSmThreads / kWave) + threadIdx.x / kWave;
    const uint32_t row = wave * RPW + lane / TL;
    const uint32_t j = lane % TL;
    const bool live = row < rows;
    const size_t row_base = (size_t)min(row, rows - 1) * row_vecs;
    const u32x4 *in = reinterpret_cast<const u32x4 *>(x) + row_base;
    u32x4 *out = reinterpret_cast<u32x4 *>(y) + row_base;
    u32x4 raw[VPL];
#pragma unroll
    for (int v = 0; v < VPL; v++) raw[v] = load_stream(in + min(v * TL + j, row_vecs - 1));
    float f[VPL][EPV];
    float mx = kNegInf;
#pragma unroll
    for (int v = 0; v < VPL; v++) {
        Store<T>::unpack(raw[v], f[v]);
        const bool have = v * TL + j < row_vecs;
#pragma unroll
        for (int e = 0; e < EPV; e++) {
            f[v][e] = have ? f[v][e] : kNegInf;  // padding: exp gives 0
            mx = fmaxf(mx, f[v][e]);
        }
    }
    float shift = 0.0f;
    if (stable) {
        shift = team_max<TL>(mx);
        shift = shift == kNegInf ? 0.0f : shift;  // a row of -inf: keep the reference's 0/0
    }
    const float bias = -shift * kLog2e;
    float total = 0.0f;
#pragma unroll
    for (int v = 0; v < VPL; v++)
#pragma unroll
        for (int e = 0; e < EPV; e++) {
            f[v][e] = __builtin_amdgcn_exp2f(fmaf(f[v][e], kLog2e, bias));
            total += f[v][e];
        }
    total = team_sum<TL>(total);
    const float inv = 1.0f / total;
#pragma unroll
    for (int v = 0; v < VPL; v++) {
#pragma unroll
        for (int e = 0; e < EPV; e++) f[v][e] *= inv;
        if (live && v * TL + j < row_vecs) store_stream(out + v * TL + j, Store<T>::pack(f[v]));
    }
}

// Any row length / alignment: one wavefront per row, lane-strided elements, the row
// re-read from cache for each of the (up to) three passes.
template <typename T>
__global__ __launch_bounds__(kSmThreads) void softmax_generic_kernel(const T *x, T *y, uint32_t rows,
                                                                     uint32_t cols, int stable) {
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t row = blockIdx.x * (kSmThreads / kWave) + threadIdx.x / kWave;
    if (row >= rows) return;
    const T *in = x + (size_t)row * cols;
    T *out = y + (size_t)row * cols;
    float shift = 0.0f;
    if (stable) {
        float mx = kNegInf;
        for (uint32_t c = lane; c < cols; c += kWave) mx = fmaxf(mx, Store<T>::load1(in + c));
        mx = team_max<64>(mx);
        shift = mx == kNegInf ? 0.0f : mx;
    }
    const float bias = -shift * kLog2e;
    float total = 0.0f;
    for (uint32_t c = lane; c < cols; c += kWave)
        total += __builtin_amdgcn_exp2f(fmaf(Store<T>::load1(in + c), kLog2e, bias));
    total = wave_sum(total);
    const float inv = 1.0f / total;
    // in place: every element of the row has been read by now, and a lane rewrites only
    // the elements it reads itself in this pass
    for (uint32_t c = lane; c < cols; c += kWave) {
        const float e = __builtin_amdgcn_exp2f(fmaf(Store<T>::load1(in + c), kLog2e, bias));
        Store<T>::store1(out + c, e * inv);
    }
}

// Short rows without alignment (77 text tokens): the whole row in ITERS registers per
// lane, one read and one write per element.
template <typename T, int ITERS>
__global__ __launch_bounds__(kSmThreads) void softmax_short_kernel(const T *x, T *y, uint32_t rows,
                                                                   uint32_t cols, int stable) {
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t row = blockIdx.x * (kSmThreads / kWave) + threadIdx.x / kWave;
    if (row >= rows) return;
    const T *in = x + (size_t)row * cols;
    T *out = y + (size_t)row * cols;
    float f[ITERS];
    float mx = kNegInf;
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        const uint32_t c = lane + i * kWave;
        const float v = Store<T>::load1(in + min(c, cols - 1));
        f[i] = c < cols ? v : kNegInf;
        mx = fmaxf(mx, f[i]);
    }
    float shift = 0.0f;
    if (stable) {
        mx = team_max<64>(mx);
        shift = mx == kNegInf ? 0.0f : mx;
    }
    const float bias = -shift * kLog2e;
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        f[i] = __builtin_amdgcn_exp2f(fmaf(f[i], kLog2e, bias));
        total += f[i];
    }
    total = wave_sum(total);
    const float inv = 1.0f / total;
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        const uint32_t c = lane + i * kWave;
        if (c < cols) Store<T>::store1(out + c, f[i] * inv);
    }
}

// ---------------------------------------------------------------------------
// DDIM update (eta = 0): the three float loops of the replaced host code as one pass,
// with individually rounded operations in the same order, so float32 storage gives
// the host loop's bits.
// ---------------------------------------------------------------------------
constexpr int kDdimThreads = 256;

struct DdimCoef {
    float sqrt_one_minus_at, sqrt_at, sqrt_one_minus_aprev, sqrt_aprev;
};

__device__ __forceinline__ float ddim_one(float x, float e, const DdimCoef &c) {
#pragma clang fp contract(off)  // no fused multiply-add: each product is rounded before it is added
    const float scaled = c.sqrt_one_minus_at * e;
    const float pred_x0 = (x - scaled) / c.sqrt_at;  // IEEE division (hipcc's default for float)
    const float dir_xt = c.sqrt_one_minus_aprev * e;
    const float back = c.sqrt_aprev * pred_x0;
    return back + dir_xt;
}

template <typename T>
__global__ __launch_bounds__(kDdimThreads) void ddim_update_kernel(const T *x, const T *e_t, T *x_prev,
                                                                   size_t n, int vectors, DdimCoef c) {
    constexpr int EPV = Store<T>::EPV;
    const size_t stride = (size_t)gridDim.x * kDdimThreads;
    const size_t first = (size_t)blockIdx.x * kDdimThreads + threadIdx.x;
    if (vectors) {
        const size_t vecs = n / EPV;
        for (size_t v = first; v < vecs; v += stride) {
            float a[EPV], b[EPV], r[EPV];
            Store<T>::unpack(reinterpret_cast<const u32x4 *>(x)[v], a);
            Store<T>::unpack(reinterpret_cast<const u32x4 *>(e_t)[v], b);
#pragma unroll
            for (int i = 0; i < EPV; i++) r[i] = ddim_one(a[i], b[i], c);
            reinterpret_cast<u32x4 *>(x_prev)[v] = Store<T>::pack(r);
        }
        for (size_t i = vecs * EPV + first; i < n; i += stride)
            Store<T>::store1(x_prev + i, ddim_one(Store<T>::load1(x + i), Store<T>::load1(e_t + i), c));
    } else {
        for (size_t i = first; i < n; i += stride)
            Store<T>::store1(x_prev + i, ddim_one(Store<T>::load1(x + i), Store<T>::load1(e_t + i), c));
    }
}

template <typename T, int M>
void linear_launch(const T *x, const T *w, const float *bias, T *y, uint32_t m, uint32_t n, uint32_t k,
                   int act_in, int act_out, hipStream_t stream) {
    constexpr int EPV = Store<T>::EPV;
    const uint32_t blocks = (n + kLinWaves - 1) / kLinWaves;
    hipLaunchKernelGGL((linear_rows_kernel<T, M>), dim3(blocks), dim3(kLinThreads),
                       (size_t)M * k * sizeof(float), stream, x, w, bias, y, m, n, k / EPV, act_in,
                       act_out);
}

template <typename T, int VPL, int TL>
void softmax_team_launch(const T *x, T *y, uint32_t rows, uint32_t row_vecs, int stable,
                         hipStream_t stream) {
    constexpr uint32_t rows_per_block = (kSmThreads / kWave) * (kWave / TL);
    hipLaunchKernelGGL((softmax_team_kernel<T, VPL, TL>), dim3((rows + rows_per_block - 1) / rows_per_block),
                       dim3(kSmThreads), 0, stream, x, y, rows, row_vecs, stable);
}

}  // namespace

template <typename T>
int linear_rows_dispatch(const void *xv, const void *wv, const float *bias, void *yv, size_t m,
                         size_t n, size_t k, int act_in, int act_out, hipStream_t stream) {
    constexpr int EPV = Store<T>::EPV;
    const T *x = static_cast<const T *>(xv);
    const T *w = static_cast<const T *>(wv);
    T *y = static_cast<T *>(yv);
    if (m == 0 || n == 0) return MSD_OK;
    if (m > 8 || n > 0x7FFFFFFFull / kLinWaves || k > 0x7FFFFFFFull) return MSD_ERR_INVALID_VALUE;
    const uint32_t m_pad = m <= 1 ? 1 : m <= 2 ? 2 : m <= 4 ? 4 : 8;
    const bool staged = k != 0 && k % EPV == 0 && aligned16(x) && aligned16(w) &&
                        (size_t)m_pad * k <= kLinMaxStaged;
    if (staged) {
        switch (m_pad) {
            case 1: linear_launch<T, 1>(x, w, bias, y, (uint32_t)m, (uint32_t)n, (uint32_t)k, act_in, act_out, stream); break;
            case 2: linear_launch<T, 2>(x, w, bias, y, (uint32_t)m, (uint32_t)n, (uint32_t)k, act_in, act_out, stream); break;
            case 4: linear_launch<T, 4>(x, w, bias, y, (uint32_t)m, (uint32_t)n, (uint32_t)k, act_in, act_out, stream); break;
            default: linear_launch<T, 8>(x, w, bias, y, (uint32_t)m, (uint32_t)n, (uint32_t)k, act_in, act_out, stream); break;
        }
    } else {
        const uint32_t blocks = (uint32_t)((n + kLinWaves - 1) / kLinWaves);
        hipLaunchKernelGGL((linear_rows_generic_kernel<T>), dim3(blocks), dim3(kLinThreads), 0, stream, x,
                           w, bias, y, (uint32_t)m, (uint32_t)n, (uint32_t)k, act_in, act_out);
    }
    return launch_status();
}

template <typename T>
int softmax_dispatch(const void *xv, void *yv, size_t rows, size_t cols, int stable, hipStream_t stream) {
    constexpr int EPV = Store<T>::EPV;
    const T *x = static_cast<const T *>(xv);
    T *y = static_cast<T *>(yv);
    if (rows == 0 || cols == 0) return MSD_OK;
    constexpr size_t waves_per_block = kSmThreads / kWave;
    if (rows > 0x7FFFFFFFull || cols > 0x7FFFFFFFull) return MSD_ERR_INVALID_VALUE;
    const uint32_t r = (uint32_t)rows, c = (uint32_t)cols;
    const size_t row_vecs = cols / EPV;
    const bool vec_ok = cols % EPV == 0 && aligned16(x) && aligned16(y) && row_vecs <= 1024;
    if (vec_ok) {
        const uint32_t rv = (uint32_t)row_vecs;
        if (rv <= 8) softmax_team_launch<T, 1, 8>(x, y, r, rv, stable, stream);
        else if (rv <= 16) softmax_team_launch<T, 2, 8>(x, y, r, rv, stable, stream);
        else if (rv <= 32) softmax_team_launch<T, 4, 8>(x, y, r, rv, stable, stream);
        else if (rv <= 64) softmax_team_launch<T, 1, 64>(x, y, r, rv, stable, stream);
        else if (rv <= 128) softmax_team_launch<T, 2, 64>(x, y, r, rv, stable, stream);
        else if (rv <= 256) softmax_team_launch<T, 4, 64>(x, y, r, rv, stable, stream);
        else if (rv <= 512) softmax_team_launch<T, 8, 64>(x, y, r, rv, stable, stream);
        else softmax_team_launch<T, 16, 64>(x, y, r, rv, stable, stream);
        return launch_status();
    }
    const dim3 grid((uint32_t)((rows + waves_per_block - 1) / waves_per_block));
    if (cols <= 2 * kWave)
        hipLaunchKernelGGL((softmax_short_kernel<T, 2>), grid, dim3(kSmThreads), 0, stream, x, y, r, c, stable);
    else if (cols <= 8 * kWave)
        hipLaunchKernelGGL((softmax_short_kernel<T, 8>), grid, dim3(kSmThreads), 0, stream, x, y, r, c, stable);
    else
        hipLaunchKernelGGL((softmax_generic_kernel<T>), grid, dim3(kSmThreads), 0, stream, x, y, r, c, stable);
    return launch_status();
}

template <typename T>
int ddim_update_dispatch(const void *xv, const void *ev, void *yv, size_t n, float a_t, float a_prev,
                         float sqrt_one_minus_at, hipStream_t stream) {
    if (n == 0) return MSD_OK;
    DdimCoef c;
    c.sqrt_one_minus_at = sqrt_one_minus_at;
    c.sqrt_at = sqrtf(a_t);  // correctly rounded on the host, as in the replaced loop
    c.sqrt_one_minus_aprev = sqrtf(1.0f - a_prev);
    c.sqrt_aprev = sqrtf(a_prev);
    const int vectors = aligned16(xv) && aligned16(ev) && aligned16(yv);
    const size_t want = (n / Store<T>::EPV + kDdimThreads) / kDdimThreads;
    hipLaunchKernelGGL((ddim_update_kernel<T>), dim3((uint32_t)(want < 4096 ? want : 4096)),
                       dim3(kDdimThreads), 0, stream, static_cast<const T *>(xv),
                       static_cast<const T *>(ev), static_cast<T *>(yv), n, vectors, c);
    return launch_status();
}

template int linear_rows_dispatch<float>(const void *, const void *, const float *, void *, size_t, size_t, size_t, int, int, hipStream_t);
template int linear_rows_dispatch<__half>(const void *, const void *, const float *, void *, size_t, size_t, size_t, int, int, hipStream_t);
template int softmax_dispatch<float>(const void *, void *, size_t, size_t, int, hipStream_t);
template int softmax_dispatch<__half>(const void *, void *, size_t, size_t, int, hipStream_t);
template int ddim_update_dispatch<float>(const void *, const void *, void *, size_t, float, float, float, hipStream_t);
template int ddim_update_dispatch<__half>(const void *, const void *, void *, size_t, float, float, float, hipStream_t);

}  // namespace msd
