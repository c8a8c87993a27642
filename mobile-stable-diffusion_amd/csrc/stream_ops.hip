// Streaming kernels for gfx950: the GEGLU epilogue, elementwise SiLU / GELU /
// quick_GELU and the sinusoidal timestep embedding.  Flat 16-byte accesses, U
// vectors per lane with every load issued before the first use; all workgroups
// but a ragged last one run branch-free.
#include "msd_device.h"
#include "msd_internal.h"

#include <cmath>
#include <type_traits>

namespace msd {
namespace {

constexpr int kStreamThreads = 256;
// GEGLU runs one wavefront per workgroup: with two loads and 21 VALU instructions per element
// in flight per lane, single-wavefront workgroups start and retire soonest (measured 4.5 %
// faster over the step's 16 launches than 256-lane workgroups; the plain copy prefers 256).
constexpr int kGegluThreads = 64;
constexpr int kStreamUnroll = 1;  // vectors per lane of the elementwise kernels

// out[r, c] = proj[r, c] * gelu(proj[r, inner + c]); vectors never straddle a row.
// Every workgroup but the last takes the branch-free path: 2*U loads in flight
// per lane before the first use.
template <typename T, int U>
__global__ __launch_bounds__(kGegluThreads) void geglu_kernel(const T *__restrict__ proj,
                                                               T *__restrict__ out,
                                                               uint32_t out_vecs,
                                                               FastDiv vec_per_row) {
    constexpr int EPV = Store<T>::EPV;
    const u32x4 *in = reinterpret_cast<const u32x4 *>(proj);
    u32x4 *o = reinterpret_cast<u32x4 *>(out);
    const uint32_t block_base = blockIdx.x * (kGegluThreads * U);
    const uint32_t base = block_base + threadIdx.x;
    const bool full = block_base + kGegluThreads * U <= out_vecs;  // uniform
    u32x4 va[U], vb[U];
    uint32_t ovs[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const uint32_t ov = base + u * kGegluThreads;
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
        if (full || base + u * kGegluThreads < out_vecs) store_stream(o + ovs[u], packed);
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
template <typename T, typename OP, int U>
__global__ __launch_bounds__(kStreamThreads) void act_kernel(const T *x, T *y, uint32_t vecs,
                                                             size_t n) {
    constexpr int EPV = Store<T>::EPV;
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

// c[i] = a[i] + b[i]  (chunk_vecs == 0), or c[i] = a[i] + b[i / chunk] with one b value per
// chunk of `chunk_vecs` vectors (the per-channel broadcast add).  c may alias a or b.
template <typename T>
__global__ __launch_bounds__(kStreamThreads) void add_kernel(const T *a, const T *b, T *c,
                                                             uint32_t vecs, FastDiv chunk_vecs) {
    constexpr int EPV = Store<T>::EPV;
    const uint32_t v = blockIdx.x * kStreamThreads + threadIdx.x;
    if (v >= vecs) return;
    float fa[EPV], fb[EPV];
    Store<T>::unpack(load_stream(reinterpret_cast<const u32x4 *>(a) + v), fa);
    if (chunk_vecs.d == 0) {
        Store<T>::unpack(load_stream(reinterpret_cast<const u32x4 *>(b) + v), fb);
#pragma unroll
        for (int e = 0; e < EPV; e++) fa[e] += fb[e];
    } else {
        const float bv = Store<T>::load1(b + fast_div(v, chunk_vecs));
#pragma unroll
        for (int e = 0; e < EPV; e++) fa[e] += bv;
    }
    store_stream(reinterpret_cast<u32x4 *>(c) + v, Store<T>::pack(fa));
}

template <typename T>
__global__ __launch_bounds__(kStreamThreads) void add_generic_kernel(const T *a, const T *b, T *c,
                                                                     size_t n, size_t chunk_size) {
    for (size_t i = (size_t)blockIdx.x * kStreamThreads + threadIdx.x; i < n;
         i += (size_t)gridDim.x * kStreamThreads) {
        const float bv = Store<T>::load1(b + (chunk_size ? i / chunk_size : i));
        Store<T>::store1(c + i, Store<T>::load1(a + i) + bv);
    }
}

// ---------------------------------------------------------------------------
// [i, j, k] -> [i, k, j] through a 64 x 64 LDS tile: reads run along k, writes along j, both in
// 4-element pieces (8 or 16 bytes), tile rows padded by one piece against bank conflicts.
// ---------------------------------------------------------------------------
constexpr int kTile = 64;

template <typename T>
__global__ __launch_bounds__(256) void permute_021_kernel(const T *__restrict__ src,
                                                          T *__restrict__ dst, uint32_t jsize,
                                                          uint32_t ksize) {
    typedef T vec4 __attribute__((ext_vector_type(4)));
    __shared__ T tile[kTile][kTile + 4];
    const uint32_t k0 = blockIdx.x * kTile, j0 = blockIdx.y * kTile, i = blockIdx.z;
    const T *in = src + (size_t)i * jsize * ksize;
    T *out = dst + (size_t)i * jsize * ksize;
    const uint32_t lane4 = (threadIdx.x & 15) * 4, row = threadIdx.x >> 4;  // 16 rows per pass
#pragma unroll
    for (int pass = 0; pass < 4; pass++) {
        const uint32_t j = j0 + row + pass * 16, k = k0 + lane4;
        if (j < jsize && k < ksize) {  // jsize, ksize are multiples of 4: a piece is all in or out
            const vec4 v = *reinterpret_cast<const vec4 *>(in + (size_t)j * ksize + k);
#pragma unroll
            for (int e = 0; e < 4; e++) tile[row + pass * 16][lane4 + e] = v[e];
        }
    }
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < 4; pass++) {
        const uint32_t k = k0 + row + pass * 16, j = j0 + lane4;
        if (k < ksize && j < jsize) {
            vec4 v;
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = tile[lane4 + e][row + pass * 16];
            *reinterpret_cast<vec4 *>(out + (size_t)k * jsize + j) = v;
        }
    }
}

// The same permute with 16-byte accesses on both sides and an LDS tile of 32-bit words that is
// written transposed: word w of tile row k belongs to output row k (one 4-byte element, or the
// 2-byte elements of input rows 2w and 2w + 1 at column k, paired in registers after the load).
// Inside a tile row the aligned groups of four words are permuted by an XOR with a number taken
// from the row index, chosen so that the 32 lanes of a half wavefront, which write one column each
// (8 rows a fixed distance apart x 4 adjacent words), fall on 32 different banks, while a lane's
// four output words stay adjacent and aligned: the read side is one 16-byte LDS access per piece,
// and the eight lanes that read one tile row together take eight different groups.
// ES = bytes per element; a workgroup moves 64 x 64 elements; jsize and ksize are multiples of
// 16 / ES (host), so a 16-byte piece is all inside the tensor or all outside.
template <int ES, bool JFAST>
__global__ __launch_bounds__(256) void permute_021_words_kernel(const void *__restrict__ srcv,
                                                                void *__restrict__ dstv, uint32_t jsize,
                                                                uint32_t ksize) {
    constexpr uint32_t kWords = kTile * ES / 4;   // 32-bit words per output row of the tile: 32 or 64
    constexpr uint32_t kRowShift = ES == 4 ? 2 : 3;  // tile rows one lane writes: 4 or 8
    __shared__ u32x4 tile4[kTile * kWords / 4];
    uint32_t *tile = reinterpret_cast<uint32_t *>(tile4);
    // word `col` of tile row `row` lives at this index
    auto at = [](uint32_t row, uint32_t col) { return row * kWords + (col ^ (((row >> kRowShift) & 7u) << 2)); };
    // JFAST: consecutive workgroups take consecutive tiles of one output row
    const uint32_t k0 = (JFAST ? blockIdx.y : blockIdx.x) * kTile, j0 = (JFAST ? blockIdx.x : blockIdx.y) * kTile;
    const uint32_t i = blockIdx.z;
    const size_t plane = (size_t)i * jsize * ksize;  // in elements
    const char *in = static_cast<const char *>(srcv) + plane * ES;
    char *out = static_cast<char *>(dstv) + plane * ES;
    const uint32_t t = threadIdx.x;
    if (ES == 4) {
        // a lane loads elements k .. k+3 of one input row, four times: 8 lanes cover 32 columns,
        // the passes take the two column halves of the tile and the two halves of its rows.  All
        // loads leave before the first LDS write (a piece outside the tensor re-reads the plane's
        // first piece instead of sitting behind a branch).
        const uint32_t kq = (t & 7) * 4, jr = t >> 3;
        u32x4 v[4];
#pragma unroll
        for (int pass = 0; pass < 4; pass++) {
            const uint32_t k = k0 + kq + 32 * (pass & 1), j = j0 + jr + 32 * (pass >> 1);
            const size_t from = (j < jsize && k < ksize) ? ((size_t)j * ksize + k) * 4 : 0;
            v[pass] = load_stream(reinterpret_cast<const u32x4 *>(in + from));
        }
#pragma unroll
        for (int pass = 0; pass < 4; pass++) {
            const uint32_t kl = kq + 32 * (pass & 1), jl = jr + 32 * (pass >> 1);
            if (j0 + jl < jsize && k0 + kl < ksize) {
#pragma unroll
                for (int e = 0; e < 4; e++) tile[at(kl + e, jl)] = v[pass][e];
            }
        }
    } else {
        // a lane loads elements k .. k+7 of input rows j and j+1 and pairs them by column
        const uint32_t kq = (t & 7) * 8, jw = t >> 3;  // jw: word of the output rows, 0 .. 31
        const uint32_t j = j0 + 2 * jw, k = k0 + kq;
        if (j < jsize && k < ksize) {  // (jsize is even: row j + 1 exists)
            const u32x4 a = load_stream(reinterpret_cast<const u32x4 *>(in + ((size_t)j * ksize + k) * 2));
            const u32x4 b = load_stream(reinterpret_cast<const u32x4 *>(in + ((size_t)(j + 1) * ksize + k) * 2));
#pragma unroll
            for (int w = 0; w < 4; w++) {
                tile[at(kq + 2 * w, jw)] = (a[w] & 0xffffu) | (b[w] << 16);
                tile[at(kq + 2 * w + 1, jw)] = (a[w] >> 16) | (b[w] & 0xffff0000u);
            }
        }
    }
    __syncthreads();
    // a lane stores 16-byte pieces (four words) of output rows; all LDS reads come first
    constexpr uint32_t kPieces = kWords / 4;          // pieces per output row of the tile: 8 or 16
    constexpr uint32_t kRowsPerPass = 256 / kPieces;  // 32 or 16
    constexpr uint32_t kPasses = kTile / kRowsPerPass;
    const uint32_t wq = (t % kPieces) * 4, kr = t / kPieces;
    u32x4 w[kPasses];
#pragma unroll
    for (uint32_t pass = 0; pass < kPasses; pass++)  // (pieces outside the tensor are read but never stored)
        w[pass] = tile4[at(kr + pass * kRowsPerPass, wq) / 4];
#pragma unroll
    for (uint32_t pass = 0; pass < kPasses; pass++) {
        const uint32_t k = k0 + kr + pass * kRowsPerPass, j = j0 + wq * (4 / ES);
        if (k < ksize && j < jsize) store_stream(reinterpret_cast<u32x4 *>(out + ((size_t)k * jsize + j) * ES), w[pass]);
    }
}

template <typename T>
__global__ __launch_bounds__(kStreamThreads) void permute_021_generic_kernel(
    const T *__restrict__ src, T *__restrict__ dst, size_t isize, size_t jsize, size_t ksize) {
    const size_t n = isize * jsize * ksize;
    for (size_t d = (size_t)blockIdx.x * kStreamThreads + threadIdx.x; d < n;
         d += (size_t)gridDim.x * kStreamThreads) {
        const size_t j = d % jsize, k = (d / jsize) % ksize, i = d / (jsize * ksize);
        dst[d] = src[(i * jsize + j) * ksize + k];
    }
}

// ---------------------------------------------------------------------------
// Timestep embedding
// ---------------------------------------------------------------------------
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

// ---- streaming dispatch ----------------------------------------------------
inline uint32_t stream_blocks(size_t vecs, int unroll) {
    const size_t per_block = (size_t)kStreamThreads * unroll;
    return (uint32_t)((vecs + per_block - 1) / per_block);
}

}  // namespace

template <typename T>
int geglu_dispatch(const void *pv, void *ov, size_t rows, size_t inner, hipStream_t stream) {
    constexpr int EPV = Store<T>::EPV;
    const T *proj = static_cast<const T *>(pv);
    T *out = static_cast<T *>(ov);
    if (rows == 0 || inner == 0) return MSD_OK;
    const size_t out_vecs = rows * (inner / EPV);
    if (aligned16(proj) && aligned16(out) && inner % EPV == 0 && out_vecs < 0x7FFFFFFFull &&
        rows < 0x7FFFFFFFull) {
        const FastDiv fd = make_fast_div((uint32_t)(inner / EPV));
        // one vector per lane: these launches are short enough that a lane's dependent ALU chain
        // is on the critical path, and more, lighter wavefronts overlap it with other loads
        // (measured 9 - 30 % faster than 4 vectors per lane at every UNet shape)
        const int tune_vectors = g_tuning.geglu_vectors.load(std::memory_order_relaxed);
        const int unroll = tune_vectors ? tune_vectors : 1;
        const uint32_t ov = (uint32_t)out_vecs;
        auto blocks = [&](int u) { return (uint32_t)((out_vecs + kGegluThreads * u - 1) / (kGegluThreads * u)); };
        if (unroll == 1)
            launch((geglu_kernel<T, 1>), dim3(blocks(1)), dim3(kGegluThreads), 0, stream, proj, out, ov, fd);
        else if (unroll == 2)
            launch((geglu_kernel<T, 2>), dim3(blocks(2)), dim3(kGegluThreads), 0, stream, proj, out, ov, fd);
        else
            launch((geglu_kernel<T, 4>), dim3(blocks(4)), dim3(kGegluThreads), 0, stream, proj, out, ov, fd);
    } else {
        const size_t n = rows * inner;
        const size_t want = (n + kStreamThreads - 1) / kStreamThreads;
        launch((geglu_generic_kernel<T>), dim3((uint32_t)(want < 65536 ? want : 65536)),
                           dim3(kStreamThreads), 0, stream, proj, out, rows, inner);
    }
    return launch_status();
}

namespace {

template <typename T, typename OP>
int act_launch(const void *xv, void *yv, size_t n, hipStream_t stream) {
    constexpr int EPV = Store<T>::EPV;
    const T *x = static_cast<const T *>(xv);
    T *y = static_cast<T *>(yv);
    if (n == 0) return MSD_OK;
    const size_t vecs = n / EPV;
    if (aligned16(x) && aligned16(y) && vecs < 0x7FFFFFFFull) {
        const int tune_vectors = g_tuning.act_vectors.load(std::memory_order_relaxed);
        const int unroll = tune_vectors ? tune_vectors : kStreamUnroll;
        const uint32_t blocks = vecs ? stream_blocks(vecs, unroll) : 1u;
        if (unroll == 4)
            launch((act_kernel<T, OP, 4>), dim3(blocks), dim3(kStreamThreads), 0, stream, x, y,
                               (uint32_t)vecs, n);
        else if (unroll == 2)
            launch((act_kernel<T, OP, 2>), dim3(blocks), dim3(kStreamThreads), 0, stream, x, y,
                               (uint32_t)vecs, n);
        else
            launch((act_kernel<T, OP, 1>), dim3(blocks), dim3(kStreamThreads), 0, stream, x, y,
                               (uint32_t)vecs, n);
    } else {
        const size_t want = (n + kStreamThreads - 1) / kStreamThreads;
        launch((act_generic_kernel<T, OP>),
                           dim3((uint32_t)(want < 65536 ? want : 65536)), dim3(kStreamThreads), 0,
                           stream, x, y, n);
    }
    return launch_status();
}


}  // namespace

template <typename T>
int add_dispatch(const void *av, const void *bv, void *cv, size_t n, size_t chunk_size,
                 hipStream_t stream) {
    constexpr int EPV = Store<T>::EPV;
    const T *a = static_cast<const T *>(av);
    const T *b = static_cast<const T *>(bv);
    T *c = static_cast<T *>(cv);
    if (n == 0) return MSD_OK;
    const bool vec_ok = aligned16(a) && aligned16(c) && n % EPV == 0 && n / EPV < 0x7FFFFFFFull &&
                        (chunk_size == 0 ? aligned16(b) : chunk_size % EPV == 0);
    if (vec_ok) {
        const uint32_t vecs = (uint32_t)(n / EPV);
        FastDiv fd = make_fast_div((uint32_t)(chunk_size / EPV));
        if (chunk_size == 0) fd.d = 0;
        launch((add_kernel<T>), dim3((vecs + kStreamThreads - 1) / kStreamThreads),
                           dim3(kStreamThreads), 0, stream, a, b, c, vecs, fd);
    } else {
        const size_t want = (n + kStreamThreads - 1) / kStreamThreads;
        launch((add_generic_kernel<T>), dim3((uint32_t)(want < 65536 ? want : 65536)),
                           dim3(kStreamThreads), 0, stream, a, b, c, n, chunk_size);
    }
    return launch_status();
}

template <typename TT>
int permute_021_dispatch(const void *srcv, void *dstv, size_t isize, size_t jsize, size_t ksize,
                         hipStream_t stream) {
    // pure data movement: elements are handled as raw 16- or 32-bit words
    typedef typename std::conditional<sizeof(TT) == 2, uint16_t, uint32_t>::type T;
    const T *src = static_cast<const T *>(srcv);
    T *dst = static_cast<T *>(dstv);
    if (isize * jsize * ksize == 0) return MSD_OK;
    const uintptr_t piece = 4 * sizeof(T);
    const bool tiled = jsize % 4 == 0 && ksize % 4 == 0 && reinterpret_cast<uintptr_t>(src) % piece == 0 &&
                       reinterpret_cast<uintptr_t>(dst) % piece == 0 && isize <= 65535 &&
                       (jsize + kTile - 1) / kTile <= 65535 && ksize < 0x7FFFFFFFull && jsize < 0x7FFFFFFFull;
    const size_t epv = 16 / sizeof(T);
    const bool words = tiled && jsize % epv == 0 && ksize % epv == 0 && aligned16(src) && aligned16(dst);
    const dim3 tiles((uint32_t)((ksize + kTile - 1) / kTile), (uint32_t)((jsize + kTile - 1) / kTile), (uint32_t)isize);
    // Output rows shorter than input rows: consecutive workgroups take the tiles of one output
    // row, so that its 128-byte pieces are written at about the same time (batch 32, 320 x 4096
    // -> 4096 x 320, fp16: 29.9 us against 32.1 with consecutive tiles along the input rows; the
    // copy takes 29.1; the other way round nothing changes).
    const bool jfast = jsize < ksize;
    if (words && jfast && tiles.x <= 65535) {
        launch((permute_021_words_kernel<(int)sizeof(T), true>), dim3(tiles.y, tiles.x, tiles.z), dim3(256), 0,
                           stream, srcv, dstv, (uint32_t)jsize, (uint32_t)ksize);
    } else if (words) {
        launch((permute_021_words_kernel<(int)sizeof(T), false>), tiles, dim3(256), 0, stream, srcv, dstv,
                           (uint32_t)jsize, (uint32_t)ksize);
    } else if (tiled) {
        launch((permute_021_kernel<T>),
                           dim3((uint32_t)((ksize + kTile - 1) / kTile), (uint32_t)((jsize + kTile - 1) / kTile),
                                (uint32_t)isize),
                           dim3(256), 0, stream, src, dst, (uint32_t)jsize, (uint32_t)ksize);
    } else {
        const size_t want = (isize * jsize * ksize + kStreamThreads - 1) / kStreamThreads;
        launch((permute_021_generic_kernel<T>), dim3((uint32_t)(want < 65536 ? want : 65536)),
                           dim3(kStreamThreads), 0, stream, src, dst, isize, jsize, ksize);
    }
    return launch_status();
}

template <typename T>
int act_dispatch(Act op, const void *x, void *y, size_t n, hipStream_t stream) {
    switch (op) {
        case Act::Silu: return act_launch<T, OpSilu>(x, y, n, stream);
        case Act::Gelu: return act_launch<T, OpGelu>(x, y, n, stream);
        case Act::QuickGelu: return act_launch<T, OpQuickGelu>(x, y, n, stream);
        case Act::Copy: return act_launch<T, OpCopy>(x, y, n, stream);
    }
    return MSD_ERR_INVALID_VALUE;
}

template <typename T>
int temb_dispatch(const int64_t *timesteps, void *out, size_t batch, size_t dim, float max_period,
                  hipStream_t stream) {
    const uint32_t half = (uint32_t)(dim / 2);
    const uint32_t blocks = (uint32_t)((batch * half + 255) / 256);
    const float neg_log_period = -logf(max_period);  // host float log, as in the replaced host loop
    launch((timestep_embedding_kernel<T>), dim3(blocks), dim3(256), 0, stream, timesteps,
                       static_cast<T *>(out), (uint32_t)batch, half, neg_log_period);
    return launch_status();
}

template int geglu_dispatch<float>(const void *, void *, size_t, size_t, hipStream_t);
template int geglu_dispatch<__half>(const void *, void *, size_t, size_t, hipStream_t);
template int add_dispatch<float>(const void *, const void *, void *, size_t, size_t, hipStream_t);
template int add_dispatch<__half>(const void *, const void *, void *, size_t, size_t, hipStream_t);
template int permute_021_dispatch<float>(const void *, void *, size_t, size_t, size_t, hipStream_t);
template int permute_021_dispatch<__half>(const void *, void *, size_t, size_t, size_t, hipStream_t);
template int act_dispatch<float>(Act, const void *, void *, size_t, hipStream_t);
template int act_dispatch<__half>(Act, const void *, void *, size_t, hipStream_t);
template int temb_dispatch<float>(const int64_t *, void *, size_t, size_t, float, hipStream_t);
template int temb_dispatch<__half>(const int64_t *, void *, size_t, size_t, float, hipStream_t);

}  // namespace msd
