// Neighbours of the norm / activation path for gfx950: the Linear layers that act on
// the few rows of the time embedding (weight-streaming, one or two output columns per
// wavefront), the row softmax of the attention blocks (a row held in the registers
// of a team of lanes) and the DDIM latent update.
#include "msd_device.h"
#include "msd_internal.h"

#include <cmath>

namespace msd {
namespace {

// ---------------------------------------------------------------------------
// y[m, n] = act_out(act_in(x)[m, k] . w[n, k]^T + bias[n]) for m <= 8 rows.
// The time is the single pass over w (n*k elements) plus launch and memory latency, so
// the kernel is built to have one latency, not two in a row: a workgroup is a single
// wavefront that owns CPW columns; lane l requests 16-byte pieces l, l+64, ... of its
// weight rows and the same pieces of every x row (a few KiB that every wavefront
// reads from cache) before it uses any of them.  No LDS, no barrier.  With SiLU on the
// input each lane activates its own x pieces, and two columns share that work.
// Each lane adds its pieces in ascending k, then the M x CPW partial sums go through
// the DPP tree, so the result does not depend on the launch shape.
// ---------------------------------------------------------------------------

template <typename T, int M, int CPW, int ROUND = 0>
__device__ __forceinline__ void linear_rows_body(const T *__restrict__ x, const T *__restrict__ w,
                                                 const float *__restrict__ bias, T *__restrict__ y,
                                                 uint32_t m, uint32_t n, uint32_t kvecs, int act_in,
                                                 int act_out, uint32_t col0) {
    constexpr int EPV = Store<T>::EPV;
    // pieces per lane per round: one round covers k = 2048 (float with more than 4 rows: 1024)
    constexpr int kLinRound = ROUND != 0 ? ROUND : (sizeof(T) == 4 && M <= 4) ? 8 : 4;
    const uint32_t lane = threadIdx.x;
    const u32x4 *xin = reinterpret_cast<const u32x4 *>(x);
    const u32x4 *win = reinterpret_cast<const u32x4 *>(w);
    float acc[CPW][M];
#pragma unroll
    for (int c = 0; c < CPW; c++)
#pragma unroll
        for (int i = 0; i < M; i++) acc[c][i] = 0.0f;
    for (uint32_t base = lane; base < kvecs; base += kWave * kLinRound) {
        u32x4 wraw[CPW][kLinRound], xraw[M][kLinRound];
#pragma unroll
        for (int u = 0; u < kLinRound; u++) {
            const uint32_t piece = min(base + u * kWave, kvecs - 1);
#pragma unroll
            for (int c = 0; c < CPW; c++)  // a column past the last re-reads the last one
                wraw[c][u] = load_stream(win + (size_t)min(col0 + c, n - 1) * kvecs + piece);
#pragma unroll
            for (int i = 0; i < M; i++)    // rows >= m repeat the last row
                xraw[i][u] = xin[(size_t)min((uint32_t)i, m - 1) * kvecs + piece];
        }
#pragma unroll
        for (int u = 0; u < kLinRound; u++) {
            if (base + u * kWave < kvecs) {
                float xf[M][EPV];
#pragma unroll
                for (int i = 0; i < M; i++) {
                    Store<T>::unpack(xraw[i][u], xf[i]);
                    if (act_in) {
#pragma unroll
                        for (int e = 0; e < EPV; e++) xf[i][e] = silu_f(xf[i][e]);
                    }
                }
#pragma unroll
                for (int c = 0; c < CPW; c++) {
                    float wf[EPV];
                    Store<T>::unpack(wraw[c][u], wf);
#pragma unroll
                    for (int i = 0; i < M; i++)
#pragma unroll
                        for (int e = 0; e < EPV; e++) acc[c][i] = fmaf(xf[i][e], wf[e], acc[c][i]);
                }
            }
        }
    }
#pragma unroll
    for (int c = 0; c < CPW; c++) {
        float mine = 0.0f;
#pragma unroll
        for (int i = 0; i < M; i++) {
            const float total = wave_sum(acc[c][i]);
            if (lane == (uint32_t)i) mine = total;
        }
        const uint32_t col = col0 + c;
        if (lane < m && col < n) {
            float r = mine + (bias != nullptr ? bias[col] : 0.0f);
            if (act_out) r = silu_f(r);
            Store<T>::store1(y + (size_t)lane * n + col, r);
        }
    }
}

template <typename T, int M, int CPW>
__global__ __launch_bounds__(kWave) void linear_rows_kernel(
    const T *__restrict__ x, const T *__restrict__ w, const float *__restrict__ bias,
    T *__restrict__ y, uint32_t m, uint32_t n, uint32_t kvecs, int act_in, int act_out) {
    linear_rows_body<T, M, CPW>(x, w, bias, y, m, n, kvecs, act_in, act_out, blockIdx.x * CPW);
}

// Several Linear layers on the same rows x in one launch (the per-ResBlock projections of the
// time embedding all read the same [m, k] embedding): the problems' workgroups are laid end to
// end, a workgroup finds its problem by walking the table of first workgroups (at most
// kLinGroupMax entries, passed by value with the launch), then runs the same code as a single
// launch would, so each problem's result is that of its own msd_linear_rows call bit for bit.
constexpr int kLinGroupMax = 32;
struct LinearGroup {
    const void *w[kLinGroupMax];
    const float *bias[kLinGroupMax];
    void *y[kLinGroupMax];
    uint32_t n[kLinGroupMax];
    uint32_t first_block[kLinGroupMax + 1];  // first_block[count] = number of workgroups
    uint32_t count;
};

template <typename T, int M, int CPW, int ROUND = 0>
__global__ __launch_bounds__(kWave) void linear_rows_grouped_kernel(const T *__restrict__ x, LinearGroup g,
                                                                    uint32_t m, uint32_t kvecs, int act_in,
                                                                    int act_out) {
    uint32_t p = 0;
    while (p + 1 < g.count && blockIdx.x >= g.first_block[p + 1]) p++;  // uniform: scalar loop
    linear_rows_body<T, M, CPW, ROUND>(x, static_cast<const T *>(g.w[p]), g.bias[p], static_cast<T *>(g.y[p]), m,
                                g.n[p], kvecs, act_in, act_out, (blockIdx.x - g.first_block[p]) * CPW);
}

constexpr int kLinThreads = 256;  // workgroup of the scalar kernel below
constexpr int kLinWaves = kLinThreads / kWave;

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
    const uint32_t wave = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
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

// Short rows whose length is not a multiple of a 16-byte vector (77 text tokens): a
// workgroup takes RB consecutive rows (RB a multiple of 8) as one flat, 16-byte aligned
// run of memory (such a block is a whole number of vectors for any row length), moves it
// through LDS with full vectors, and a team of 4, 8 or 16 lanes per row does the arithmetic
// on the LDS copy.
constexpr uint32_t kSmFlatMaxCols = 128;  // RB = 64: 16 or 32 KiB of LDS

template <typename T, int RB, int ITERS, int TEAM>
__global__ __launch_bounds__(RB * TEAM) void softmax_flat_kernel(const T *x, T *y, uint32_t cols, int stable) {
    constexpr int EPV = Store<T>::EPV;
    constexpr int NT = RB * TEAM;
    constexpr int UN = 4;
    // [RB][cols] in the storage type: whole vectors go in and out as they are (one 16-byte LDS
    // access per vector), only the arithmetic in between touches single elements
    extern __shared__ u32x4 tile_vec[];
    T *tile = reinterpret_cast<T *>(tile_vec);
    const uint32_t block_vecs = RB * cols / EPV;
    const size_t first = (size_t)blockIdx.x * block_vecs;
    const u32x4 *in = reinterpret_cast<const u32x4 *>(x) + first;
    u32x4 *out = reinterpret_cast<u32x4 *>(y) + first;
    for (uint32_t base = threadIdx.x; base < block_vecs; base += NT * UN) {
        u32x4 raw[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) raw[u] = load_stream(in + min(base + u * NT, block_vecs - 1));
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const uint32_t v = base + u * NT;
            if (v < block_vecs) tile_vec[v] = raw[u];
        }
    }
    __syncthreads();
    // the lane's share of its row, from LDS into registers with independent reads
    T *row = tile + (threadIdx.x / TEAM) * cols;
    const uint32_t j = threadIdx.x % TEAM;
    float f[ITERS];
    float mx = kNegInf;
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        const uint32_t c = j + i * TEAM;
        f[i] = c < cols ? Store<T>::load1(row + c) : kNegInf;
        mx = fmaxf(mx, f[i]);
    }
    float shift = 0.0f;
    if (stable) {
        mx = team_max<TEAM>(mx);
        shift = mx == kNegInf ? 0.0f : mx;
    }
    const float bias = -shift * kLog2e;
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        f[i] = __builtin_amdgcn_exp2f(fmaf(f[i], kLog2e, bias));
        total += f[i];
    }
    total = team_sum<TEAM>(total);
    const float inv = 1.0f / total;
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        const uint32_t c = j + i * TEAM;
        if (c < cols) Store<T>::store1(row + c, f[i] * inv);
    }
    __syncthreads();
    for (uint32_t v = threadIdx.x; v < block_vecs; v += NT) store_stream(out + v, tile_vec[v]);
}

template <typename T, int RB, int TEAM>
void softmax_flat_launch(const T *x, T *y, uint32_t blocks, uint32_t cols, int stable, hipStream_t stream) {
    const size_t lds = (size_t)RB * cols * sizeof(T);  // a whole number of 16-byte vectors: RB is a multiple of 8
    constexpr int kFew = (80 + TEAM - 1) / TEAM, kMany = kSmFlatMaxCols / TEAM;
    if (cols <= 80)
        launch((softmax_flat_kernel<T, RB, kFew, TEAM>), dim3(blocks), dim3(RB * TEAM), lds, stream, x, y, cols, stable);
    else
        launch((softmax_flat_kernel<T, RB, kMany, TEAM>), dim3(blocks), dim3(RB * TEAM), lds, stream, x, y, cols, stable);
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
    if (act_in)  // two columns per wavefront share the activated x
        launch((linear_rows_kernel<T, M, 2>), dim3((n + 1) / 2), dim3(kWave), 0, stream, x, w, bias,
                           y, m, n, k / EPV, act_in, act_out);
    else
        launch((linear_rows_kernel<T, M, 1>), dim3(n), dim3(kWave), 0, stream, x, w, bias, y, m, n,
                           k / EPV, act_in, act_out);
}

template <typename T, int VPL, int TL>
void softmax_team_launch(const T *x, T *y, uint32_t rows, uint32_t row_vecs, int stable,
                         hipStream_t stream) {
    // long rows (a wavefront per row, 8 or 16 vectors per lane) run as single-wavefront
    // workgroups: 3 % faster at 65536 x 4096; the shorter ones keep 256 lanes
    constexpr uint32_t threads = (TL == kWave && VPL >= 8) ? kWave : kSmThreads;
    constexpr uint32_t rows_per_block = (threads / kWave) * (kWave / TL);
    launch((softmax_team_kernel<T, VPL, TL>), dim3((rows + rows_per_block - 1) / rows_per_block),
                       dim3(threads), 0, stream, x, y, rows, row_vecs, stable);
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
    if (m > 8 || n > 0x7FFFFFFFull || k > 0x7FFFFFFFull) return MSD_ERR_INVALID_VALUE;
    const uint32_t m_pad = m <= 1 ? 1 : m <= 2 ? 2 : m <= 4 ? 4 : 8;
    const bool vectors = k != 0 && k % EPV == 0 && aligned16(x) && aligned16(w);
    if (vectors) {
        switch (m_pad) {
            case 1: linear_launch<T, 1>(x, w, bias, y, (uint32_t)m, (uint32_t)n, (uint32_t)k, act_in, act_out, stream); break;
            case 2: linear_launch<T, 2>(x, w, bias, y, (uint32_t)m, (uint32_t)n, (uint32_t)k, act_in, act_out, stream); break;
            case 4: linear_launch<T, 4>(x, w, bias, y, (uint32_t)m, (uint32_t)n, (uint32_t)k, act_in, act_out, stream); break;
            default: linear_launch<T, 8>(x, w, bias, y, (uint32_t)m, (uint32_t)n, (uint32_t)k, act_in, act_out, stream); break;
        }
    } else {
        const uint32_t blocks = (uint32_t)((n + kLinWaves - 1) / kLinWaves);
        launch((linear_rows_generic_kernel<T>), dim3(blocks), dim3(kLinThreads), 0, stream, x,
                           w, bias, y, (uint32_t)m, (uint32_t)n, (uint32_t)k, act_in, act_out);
    }
    return launch_status();
}

namespace {

template <typename T, int M>
void linear_grouped_launch(const T *x, const LinearGroup &g, uint32_t m, uint32_t k, int act_in, int act_out,
                           int cpw, hipStream_t stream) {
    constexpr int EPV = Store<T>::EPV;
    const uint32_t blocks = g.first_block[g.count];
    if (cpw == 4 && k / EPV > 128 && k / EPV <= 192)  // three pieces per lane cover the row (k = 1280: 3 % faster)
        launch((linear_rows_grouped_kernel<__half, (M <= 2 ? M : 1), 4, 3>), dim3(blocks), dim3(kWave), 0,
                           stream, reinterpret_cast<const __half *>(x), g, m, k / EPV, act_in, act_out);
    else if (cpw == 4)  // (only 2-byte elements and up to two rows: see the dispatch)
        launch((linear_rows_grouped_kernel<__half, (M <= 2 ? M : 1), 4>), dim3(blocks), dim3(kWave), 0,
                           stream, reinterpret_cast<const __half *>(x), g, m, k / EPV, act_in, act_out);
    else if (cpw == 2)
        launch((linear_rows_grouped_kernel<T, M, 2>), dim3(blocks), dim3(kWave), 0, stream, x, g, m,
                           k / EPV, act_in, act_out);
    else
        launch((linear_rows_grouped_kernel<T, M, 1>), dim3(blocks), dim3(kWave), 0, stream, x, g, m,
                           k / EPV, act_in, act_out);
}

}  // namespace

template <typename T>
int linear_rows_grouped_dispatch(const void *xv, const void *const *ws, const float *const *biases,
                                 void *const *ys, const size_t *ns, size_t count, size_t m, size_t k,
                                 int act_in, int act_out, hipStream_t stream) {
    constexpr int EPV = Store<T>::EPV;
    const T *x = static_cast<const T *>(xv);
    if (m == 0 || count == 0) return MSD_OK;
    if (m > 8 || k > 0x7FFFFFFFull) return MSD_ERR_INVALID_VALUE;
    bool vectors = k != 0 && k % EPV == 0 && aligned16(x);
    for (size_t i = 0; i < count; i++) {
        if (ns[i] > 0x7FFFFFFFull) return MSD_ERR_INVALID_VALUE;
        vectors = vectors && aligned16(ws[i]);
    }
    if (!vectors) {  // odd k or alignment: one launch of the scalar kernel per problem
        for (size_t i = 0; i < count; i++) {
            const int rc = linear_rows_dispatch<T>(xv, ws[i], biases ? biases[i] : nullptr, ys[i], m, ns[i], k,
                                                   act_in, act_out, stream);
            if (rc != MSD_OK) return rc;
        }
        return MSD_OK;
    }
    const uint32_t m_pad = m <= 1 ? 1 : m <= 2 ? 2 : m <= 4 ? 4 : 8;
    // Columns per wavefront: with SiLU on the input every wavefront activates its own copy of x, so
    // columns share that work: two as in the single launch, four when the launch is large enough
    // to fill the chip anyway: fewer, longer wavefronts also stream the weights faster, with or
    // without the activation (the 22 projections of a step, 20160 columns of fp16: 15.3 us with
    // two, 12.2 us with four, 14.6 with eight; without SiLU 13.8 us with one, 11.3 with four; a
    // single 1280-column layer is slower with four, 4.25 against 3.91 us, and 4-byte elements run
    // out of registers).  The sums do not depend on it.
    size_t total_n = 0;
    for (size_t i = 0; i < count; i++) total_n += ns[i];
    const int cpw = (sizeof(T) == 2 && m_pad <= 2 && total_n >= 8192) ? 4 : act_in ? 2 : 1;
    for (size_t base = 0; base < count; base += kLinGroupMax) {
        LinearGroup g;
        g.count = 0;
        uint32_t blocks = 0;
        for (size_t i = base; i < count && i < base + kLinGroupMax; i++) {
            if (ns[i] == 0) continue;
            const uint32_t slot = g.count++;
            g.w[slot] = ws[i];
            g.bias[slot] = biases ? biases[i] : nullptr;
            g.y[slot] = ys[i];
            g.n[slot] = (uint32_t)ns[i];
            g.first_block[slot] = blocks;
            blocks += (uint32_t)((ns[i] + cpw - 1) / cpw);
        }
        if (g.count == 0) continue;
        g.first_block[g.count] = blocks;
        switch (m_pad) {
            case 1: linear_grouped_launch<T, 1>(x, g, (uint32_t)m, (uint32_t)k, act_in, act_out, cpw, stream); break;
            case 2: linear_grouped_launch<T, 2>(x, g, (uint32_t)m, (uint32_t)k, act_in, act_out, cpw, stream); break;
            case 4: linear_grouped_launch<T, 4>(x, g, (uint32_t)m, (uint32_t)k, act_in, act_out, cpw, stream); break;
            default: linear_grouped_launch<T, 8>(x, g, (uint32_t)m, (uint32_t)k, act_in, act_out, cpw, stream); break;
        }
        const int rc = launch_status();
        if (rc != MSD_OK) return rc;
    }
    return MSD_OK;
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
        // up to 64 vectors per row: one vector per lane on the smallest team that holds the row
        // (measured against two or four vectors per lane on smaller teams at 4 ... 32 vectors per
        // row, 2048 ... 524288 rows of fp16: never slower, 25-vector rows 71 against 109 us, 4-vector
        // rows 12.9 against 17.1, 32-vector rows 2.4 against 2.7 us at 2048 rows)
        if (rv <= 4) softmax_team_launch<T, 1, 4>(x, y, r, rv, stable, stream);
        else if (rv <= 8) softmax_team_launch<T, 1, 8>(x, y, r, rv, stable, stream);
        else if (rv <= 16) softmax_team_launch<T, 1, 16>(x, y, r, rv, stable, stream);
        else if (rv <= 32) softmax_team_launch<T, 1, 32>(x, y, r, rv, stable, stream);
        else if (rv <= 64) softmax_team_launch<T, 1, 64>(x, y, r, rv, stable, stream);
        else if (rv <= 128) softmax_team_launch<T, 2, 64>(x, y, r, rv, stable, stream);
        else if (rv <= 256) softmax_team_launch<T, 4, 64>(x, y, r, rv, stable, stream);
        else if (rv <= 512) softmax_team_launch<T, 8, 64>(x, y, r, rv, stable, stream);
        else softmax_team_launch<T, 16, 64>(x, y, r, rv, stable, stream);
        return launch_status();
    }
    // The flat kernel pays two barriers and two LDS round trips; below about 12000 rows the
    // row-per-wavefront kernel is quicker (3.08 against 3.10 us at 10240 x 77, 3.26 against 3.18
    // at 12288).  Lanes per row: as many as keep the launch within the 8192 wavefronts the chip
    // holds at once (a second round of wavefronts costs more than the shorter serial chain per
    // lane gains: 16 lanes per row take 4.09 us at 32768 x 77 and 7.08 at 65536, 8 lanes 4.52 and
    // 5.76); past one round 4 lanes per row are the cheapest for up to 80 columns, 8 beyond.
    // A set knob forces the flat kernel and its rows per workgroup for any size.
    const int tune_rows = g_tuning.softmax_rows.load(std::memory_order_relaxed);
    const uint32_t team = rows <= 32768 ? 16u : rows <= 65536 ? 8u : cols <= 80 ? 4u : 8u;
    // workgroups of 512 lanes up to 80 columns, of 256 beyond, and at most 64 rows
    const uint32_t lanes = cols <= 80 ? 512u : 256u;
    const uint32_t rb = tune_rows ? (uint32_t)tune_rows : lanes / team > 64u ? 64u : lanes / team;
    const bool flat_pays = tune_rows ? rows >= rb : rows >= 12288;
    if (cols <= kSmFlatMaxCols && cols >= 8 && flat_pays && aligned16(x) && aligned16(y)) {
        // whole blocks of rb rows through the flat kernel, the rest (if any) row by row below
        const uint32_t blocks = r / rb;
        switch (team * 100 + rb) {
            case 464: softmax_flat_launch<T, 64, 4>(x, y, blocks, c, stable, stream); break;
            case 432: softmax_flat_launch<T, 32, 4>(x, y, blocks, c, stable, stream); break;
            case 416: softmax_flat_launch<T, 16, 4>(x, y, blocks, c, stable, stream); break;
            case 864: softmax_flat_launch<T, 64, 8>(x, y, blocks, c, stable, stream); break;
            case 832: softmax_flat_launch<T, 32, 8>(x, y, blocks, c, stable, stream); break;
            case 816: softmax_flat_launch<T, 16, 8>(x, y, blocks, c, stable, stream); break;
            case 1664: softmax_flat_launch<T, 64, 16>(x, y, blocks, c, stable, stream); break;
            case 1632: softmax_flat_launch<T, 32, 16>(x, y, blocks, c, stable, stream); break;
            default: softmax_flat_launch<T, 16, 16>(x, y, blocks, c, stable, stream); break;
        }
        const uint32_t done = blocks * rb;
        if (done == r) return launch_status();
        x += (size_t)done * c;
        y += (size_t)done * c;
        rows -= done;
    }
    const uint32_t r_left = (uint32_t)rows;
    const dim3 grid((uint32_t)((rows + waves_per_block - 1) / waves_per_block));
    if (cols <= 2 * kWave)
        launch((softmax_short_kernel<T, 2>), grid, dim3(kSmThreads), 0, stream, x, y, r_left, c, stable);
    else if (cols <= 8 * kWave)
        launch((softmax_short_kernel<T, 8>), grid, dim3(kSmThreads), 0, stream, x, y, r_left, c, stable);
    else
        launch((softmax_generic_kernel<T>), grid, dim3(kSmThreads), 0, stream, x, y, r_left, c, stable);
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
    launch((ddim_update_kernel<T>), dim3((uint32_t)(want < 4096 ? want : 4096)),
                       dim3(kDdimThreads), 0, stream, static_cast<const T *>(xv),
                       static_cast<const T *>(ev), static_cast<T *>(yv), n, vectors, c);
    return launch_status();
}

template int linear_rows_dispatch<float>(const void *, const void *, const float *, void *, size_t, size_t, size_t, int, int, hipStream_t);
template int linear_rows_dispatch<__half>(const void *, const void *, const float *, void *, size_t, size_t, size_t, int, int, hipStream_t);
template int linear_rows_grouped_dispatch<float>(const void *, const void *const *, const float *const *, void *const *,
                                                 const size_t *, size_t, size_t, size_t, int, int, hipStream_t);
template int linear_rows_grouped_dispatch<__half>(const void *, const void *const *, const float *const *, void *const *,
                                                  const size_t *, size_t, size_t, size_t, int, int, hipStream_t);
template int softmax_dispatch<float>(const void *, void *, size_t, size_t, int, hipStream_t);
template int softmax_dispatch<__half>(const void *, void *, size_t, size_t, int, hipStream_t);
template int ddim_update_dispatch<float>(const void *, const void *, void *, size_t, float, float, float, hipStream_t);
template int ddim_update_dispatch<__half>(const void *, const void *, void *, size_t, float, float, float, hipStream_t);

}  // namespace msd
