// GroupNorm (+ SiLU) for gfx950.
//
// A unit is one (sample, group): ch_per_group * hw contiguous elements of an
// NCHW tensor.  A unit is cut into `split` slices, one workgroup per slice; the
// slice stays in registers as packed 16-byte vectors for the whole kernel, so
// the tensor is read from HBM once and written once.
//
//   1. every lane issues all its loads (K vectors) before the first use;
//   2. slice mean and M2 = sum (x - slice mean)^2 from one pass of sum and sum of squares
//      over the packed registers (DPP wavefront reduction, one LDS slot per wavefront), with
//      a second, centred pass when the mean is large against the spread;
//   3. split > 1: slices publish (mean, M2) as two tagged 64-bit words, poll
//      their siblings' words, and merge with Chan's formula.  The tag is the
//      unit's launch count, read at kernel start; the last slice to finish
//      advances it, so nothing is reset between launches and a replayed graph
//      works.  All traffic is relaxed agent-scope atomics: no cache flushes.
//   4. y = fma(x - mean, rstd * gamma[c], beta[c]) (the mean folded into the offset when it
//      is small), optional SiLU, packed store.
//
// When the output lies apart from the input and the launch is small, whole units are instead
// shared by several workgroups (SHARED): each loads and reduces the whole unit (steps 1 and 2,
// the same bits in every one; the copies of the loads meet in the L2 of the XCD the writers are
// placed on) and does step 4 for its own part of the unit.  No step 3, nothing waits.
//
// Workgroups of one unit have adjacent block ids, so a waiter's siblings are
// normally dispatched together with it.  Nothing depends on that: a wait is
// bounded (about a millisecond of polls), and a slice whose sibling has not
// published by then computes that sibling's statistics itself from the
// sibling's part of the input, which no workgroup overwrites before it has
// seen every word of its unit.  The output is the same either way; a counter
// in the scratch records how often it happened.
#include <type_traits>

#include "msd_device.h"
#include "msd_internal.h"

namespace msd {

namespace {

constexpr uint32_t kGnSpinLimit = 2048;  // default poll limit: about half a microsecond per poll
constexpr int kGenericThreads = 256;

struct GnParams {
    uint32_t vec_per_unit;   // 16-byte vectors per unit
    uint32_t vec_per_slice;  // vectors per workgroup (the last slice may be shorter)
    uint32_t split;          // workgroups per unit, power of two <= kGnMaxSplit
    uint32_t split_shift;    // log2(split)
    uint32_t groups;
    uint32_t ch_per_group;
    FastDiv hw_vec;          // vectors per channel
    float eps;
    float inv_count;         // 1 / elements per unit
    uint32_t spin_limit;     // polls before a slice stops waiting for a sibling's words
    // gn_slice_kernel<..., SHARED>: `writers` workgroups per whole unit; each loads and reduces the
    // whole unit and normalises and stores one part of it
    uint32_t writers;        // power of two
    uint32_t writers_shift;  // log2(writers)
    uint32_t part_vecs;      // vectors per part, a multiple of 64 (a wavefront is inside one part or outside)
    uint32_t xcd_shift;      // the writers of a unit have block ids (1 << xcd_shift) apart: with that many XCDs they
                             // share one XCD and its L2 (units in whole rows of that many); 0: adjacent ids
};

// Sum over the workgroup (blockDim.x / 64 wavefronts); one barrier.
__device__ __forceinline__ float block_sum_rt(float v, float *slots) {
    const float w = wave_sum(v);
    const uint32_t nw = blockDim.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) slots[threadIdx.x / kWave] = w;
    __syncthreads();
    float t = 0.0f;
    for (uint32_t i = 0; i < nw; i++) t += slots[i];
    return t;
}

__device__ __forceinline__ unsigned long long tagged(uint32_t tag, float v) {
    return ((unsigned long long)tag << 32) | (unsigned long long)__float_as_uint(v);
}

// Merges the slices of one unit.  Called by every lane of the workgroup with the slice's
// (mean, M2); `epoch` is the unit's launch count as lane 0 read it at kernel start.  On return
// stats[0] = mean and stats[1] = 1/sqrt(var + eps) of the whole unit, in LDS, after a barrier.
// Slice l covers vectors [l * vec_per_slice, min(vec_per_unit, (l + 1) * vec_per_slice)).
// `read(l, i)` returns vector i of slice l as the statistics see it (after the optional addend);
// it is only used when slice l has not published within the poll limit.
template <typename T, typename Reader>
__device__ __forceinline__ void gn_exchange(const GnScratch &scratch, const GnParams &p, uint32_t unit,
                                            uint32_t slice, uint32_t epoch, float slice_mean,
                                            float slice_m2, float *stats, Reader read) {
    constexpr int EPV = Store<T>::EPV;
    const uint32_t tid = threadIdx.x;
    unsigned long long *slot_mean = scratch.slot_mean + (size_t)unit * kGnMaxSplit;
    unsigned long long *slot_m2 = scratch.slot_m2 + (size_t)unit * kGnMaxSplit;
    if (tid < kWave) {  // wavefront 0 owns the exchange; lane 0 holds the epoch
        const uint32_t tag = (uint32_t)__builtin_amdgcn_readfirstlane((int)epoch) + 1u;
        if (tid == 0) {
            __hip_atomic_store(slot_mean + slice, tagged(tag, slice_mean), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(slot_m2 + slice, tagged(tag, slice_m2), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        }
        // lane l waits for slice l
        float m_l = 0.0f, q_l = 0.0f, n_l = 0.0f;
        bool ok = true;
        if (tid < p.split) {
            unsigned long long wm, wq;
            uint32_t polls = 0;
            // A slice never gives up on its own words: they arrive without anybody's help, and
            // having read them back is what lets it store output (see below).
            const uint32_t limit = tid == slice ? 0xFFFFFFFFu : p.spin_limit;
            do {
                wm = __hip_atomic_load(slot_mean + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                wq = __hip_atomic_load(slot_m2 + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                ok = (uint32_t)(wm >> 32) == tag && (uint32_t)(wq >> 32) == tag;
                if (!ok) __builtin_amdgcn_s_sleep(1);
            } while (!ok && ++polls < limit);
            m_l = __uint_as_float((uint32_t)wm);
            q_l = __uint_as_float((uint32_t)wq);
            const uint32_t b = tid * p.vec_per_slice;
            const uint32_t e = min(p.vec_per_unit, b + p.vec_per_slice);
            n_l = (float)((e - b) * EPV);
        }
        // Slices that have not published (not dispatched yet, or starved): this wavefront
        // computes their (mean, M2) from their part of the input, two passes.  A slice stores
        // output only after it has read back every word of its unit from the memory side, its
        // own included, so what is read here is still input unless the sibling published in the
        // meantime - then its words are at the memory side before its first output store
        // leaves, and they win when they are read again after the passes.  That second read
        // must not start before the passes' loads have returned: the wait below stops the
        // memory pipeline, and as a compiler barrier the compiler, from moving it ahead.
        unsigned long long missing = __builtin_amdgcn_ballot_w64(!ok);
        if (missing != 0) {  // uniform over the wavefront
            while (missing != 0) {
                const uint32_t s = (uint32_t)__builtin_ctzll(missing);
                missing &= missing - 1;
                const uint32_t b = s * p.vec_per_slice;
                const uint32_t n = min(p.vec_per_unit, b + p.vec_per_slice) - b;
                float sum = 0.0f;
                for (uint32_t i = tid; i < n; i += kWave) {
                    float f[EPV];
                    Store<T>::unpack(read(s, i), f);
#pragma unroll
                    for (int e = 0; e < EPV; e++) sum += f[e];
                }
                const float mean_s = wave_sum(sum) / (float)(n * EPV);
                float q = 0.0f;
                for (uint32_t i = tid; i < n; i += kWave) {
                    float f[EPV];
                    Store<T>::unpack(read(s, i), f);
#pragma unroll
                    for (int e = 0; e < EPV; e++) {
                        const float d = f[e] - mean_s;
                        q = fmaf(d, d, q);
                    }
                }
                const float m2_s = wave_sum(q);
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                if (tid == s) {
                    const unsigned long long wm =
                        __hip_atomic_load(slot_mean + s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    const unsigned long long wq =
                        __hip_atomic_load(slot_m2 + s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    const bool late = (uint32_t)(wm >> 32) == tag && (uint32_t)(wq >> 32) == tag;
                    m_l = late ? __uint_as_float((uint32_t)wm) : mean_s;
                    q_l = late ? __uint_as_float((uint32_t)wq) : m2_s;
                }
            }
            if (tid == 0)
                __hip_atomic_fetch_add(scratch.fallbacks, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // Chan: mean = sum n_l mean_l / n ; M2 = sum M2_l + sum n_l (mean_l - mean)^2
        const float total_mean = wave_sum(m_l * n_l) * p.inv_count;
        const float dm = m_l - total_mean;
        const float m2 = wave_sum(fmaf(n_l * dm, dm, q_l));
        if (tid == 0) {
            stats[0] = total_mean;
            stats[1] = __builtin_amdgcn_rsqf(m2 * p.inv_count + p.eps);
        }
    }
    __syncthreads();
}

// This slice has consumed its siblings' words: it counts itself done.  Called by lane 0 of the
// workgroup after the barrier that ends gn_exchange, so that no wavefront waits for the
// counter's old value, which comes back a memory round trip later; gn_exchange_close uses it
// at the end of the kernel.
__device__ __forceinline__ uint32_t gn_exchange_arrive(const GnScratch &scratch, uint32_t unit) {
    return __hip_atomic_fetch_add(scratch.done + unit, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The last slice to arrive closes the launch: the counter goes back to zero and the unit's
// launch count advances (both visible to the next launch, which starts after this kernel).
__device__ __forceinline__ void gn_exchange_close(const GnScratch &scratch, const GnParams &p, uint32_t unit,
                                                  uint32_t epoch, uint32_t arrived_before) {
    if (arrived_before == p.split - 1) {
        __hip_atomic_store(scratch.done + unit, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(scratch.epoch + unit, epoch + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// Sum and sum of squares of a packed vector, accumulated in float32.  Half storage uses
// v_dot2_f32_f16 (both products of a register pair are exact in float32 and are added to a
// float32 accumulator; subnormal halves count), so the statistics never need an unpacked copy
// of the slice.  Two accumulator pairs (even / odd registers) halve the dependent chains.
template <typename T>
struct Moments;
template <>
struct Moments<float> {
    static __device__ __forceinline__ void add(const u32x4 &v, float (&s)[2], float (&q)[2]) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float f = __uint_as_float(v[i]);
            s[i & 1] += f;
            q[i & 1] = fmaf(f, f, q[i & 1]);
        }
    }
};
template <>
struct Moments<__half> {
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ void add(const u32x4 &v, float (&s)[2], float (&q)[2]) {
        const half2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t w = v[i];
            const half2_t h = *reinterpret_cast<const half2_t *>(&w);
            s[i & 1] = __builtin_amdgcn_fdot2(h, ones, s[i & 1], false);
            q[i & 1] = __builtin_amdgcn_fdot2(h, h, q[i & 1], false);
        }
    }
};

// |mean| <= 2 sigma: the slice's M2 may be taken from the raw moments (relative error
// below 1e-6); otherwise it is recomputed about the mean (a second pass over the registers)
constexpr float kGnFastMoments = 4.0f;
// |mean| <= 4 sigma of the whole unit: the epilogue may fold the mean into the offset
constexpr float kGnFoldMean = 16.0f;

// Mean and M2 = sum (x - mean)^2 of the workgroup's slice, held as K packed vectors per lane
// (vector k of lane t is element k * blockDim.x + t of the slice; the first n_valid count, the
// registers of the others hold zeros).  One pass gives sum and sum of squares (wavefront
// reduction by DPP, the wavefronts' partial sums meet once in LDS, every wavefront adds them
// in the same order).  M2 = sum x^2 - n mean^2 is kept when it is well conditioned; when the
// mean is large against the spread (or the slice is constant) a second pass over the registers
// sums (x - mean)^2 instead, so the result is as accurate as a two-pass variance either way.
// The choice is the same in every wavefront: they all hold bit-identical sums.
template <typename T, int K, bool FULL>
__device__ __forceinline__ void gn_slice_stats(u32x4 (&raw)[K], uint32_t n_valid, float *red_a,
                                               float *red_b, float *red_c, float &slice_mean,
                                               float &slice_m2) {
    constexpr int EPV = Store<T>::EPV;
    const uint32_t tid = threadIdx.x;
    const uint32_t nt = blockDim.x;
    const uint32_t lane = tid & (kWave - 1);
    const uint32_t nw = nt / kWave;
    float s[2] = {0.0f, 0.0f}, q[2] = {0.0f, 0.0f};
#pragma unroll
    for (int k = 0; k < K; k++) Moments<T>::add(raw[k], s, q);
    const float wave_s = wave_sum(s[0] + s[1]);
    const float wave_q = wave_sum(q[0] + q[1]);
    if (lane == 0) {
        red_a[tid / kWave] = wave_s;
        red_b[tid / kWave] = wave_q;
    }
    __syncthreads();
    const bool entry = lane < nw;
    const float sum_x = wave_sum(entry ? red_a[lane] : 0.0f);
    const float sum_xx = wave_sum(entry ? red_b[lane] : 0.0f);
    const float count = (float)(n_valid * EPV);
    slice_mean = sum_x / count;
    slice_m2 = sum_xx - sum_x * slice_mean;
    // n mean^2 <= kappa M2; false also for a negative or NaN M2
    if (!(sum_x * slice_mean <= kGnFastMoments * slice_m2)) {  // uniform over the workgroup
        float c = 0.0f;
#pragma unroll
        for (int k = 0; k < K; k++) {
            float f[EPV];
            forget(raw[k]);  // unpack here, not once for every later use (the copies would not fit)
            Store<T>::unpack(raw[k], f);
            float ck = 0.0f;
#pragma unroll
            for (int e = 0; e < EPV; e++) {
                const float d = f[e] - slice_mean;
                ck = fmaf(d, d, ck);
            }
            if (!FULL) ck = (k * nt + tid < n_valid) ? ck : 0.0f;
            c += ck;
            // one vector at a time: unpacked copies of the whole slice would not fit the registers
            __builtin_amdgcn_sched_barrier(0);
        }
        const float wave_c = wave_sum(c);
        if (lane == 0) red_c[tid / kWave] = wave_c;
        __syncthreads();
        slice_m2 = wave_sum(entry ? red_c[lane] : 0.0f);
    }
}

// FULL: every lane owns exactly K vectors (no masking anywhere).
template <typename T, int K, bool SILU, bool FULL, bool SHARED>
__device__ __forceinline__ void gn_body(const T *x, const T *chunk, T *y,
                                        const float *__restrict__ gamma,
                                        const float *__restrict__ beta, const GnScratch &scratch,
                                        const GnParams &p, uint32_t unit, uint32_t slice, uint32_t part,
                                        uint32_t v_begin, uint32_t v_end, float *red_a,
                                        float *red_b, float *red_c, float *stats, float2 *aff) {
    constexpr int EPV = Store<T>::EPV;
    const uint32_t tid = threadIdx.x;
    const uint32_t nt = blockDim.x;
    const u32x4 *xin = reinterpret_cast<const u32x4 *>(x) + (size_t)unit * p.vec_per_unit;
    u32x4 *yout = reinterpret_cast<u32x4 *>(y) + (size_t)unit * p.vec_per_unit;

    // launch count of this unit: the tag of this launch's exchange (latency hidden by the loads)
    uint32_t epoch = 0;
    if (!SHARED && p.split > 1 && tid == 0)
        epoch = __hip_atomic_load(scratch.epoch + unit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // ---- the slice goes into registers.  Lanes past the end of a ragged slice re-read its
    // last vector (a valid address) and are masked later: no load sits behind a branch.
    u32x4 raw[K];
    // Index of a lane's k-th vector inside the unit, and its address.  Both are recomputed
    // from the lane number wherever they are needed (a few instructions) instead of being kept
    // in registers per vector; `lane_again()` returns the lane number as a value the compiler
    // cannot tie to earlier computations, so it cannot decide otherwise.
    auto lane_again = [&]() {
        uint32_t t = tid;
        asm volatile("" : "+v"(t));
        return t;
    };
    auto vidx = [&](int k, uint32_t t) {
        const uint32_t v = v_begin + k * nt + t;
        return FULL ? v : min(v, v_end - 1);
    };
    auto have = [&](int k, uint32_t t) { return FULL || v_begin + k * nt + t < v_end; };
    // the address: a base that is the same for the whole workgroup (scalar registers) plus a
    // lane offset, which for a full slice is the same for every k
    auto at = [&](auto *base, int k, uint32_t t) {
        using Byte = std::conditional_t<std::is_const<std::remove_pointer_t<decltype(base)>>::value, const char, char>;
        const uint32_t offset = vidx(k, t) * (uint32_t)sizeof(u32x4);  // a unit is smaller than 4 GiB (host)
        return reinterpret_cast<decltype(base)>(reinterpret_cast<Byte *>(base) + offset);
    };
#pragma unroll
    for (int k = 0; k < K; k++) raw[k] = load_stream(at(xin, k, tid));
    const uint32_t ch0 = (unit % p.groups) * p.ch_per_group;
    // optional per-(sample, channel) addend applied before the statistics (the reference's
    // chunkwise_add pass): the sum replaces the slice in registers, rounded to the storage
    // type exactly as a separate add kernel would have stored it
    if (chunk != nullptr) {  // uniform
        const T *cb = chunk + (size_t)(unit / p.groups) * (p.groups * p.ch_per_group);
#pragma unroll
        for (int k = 0; k < K; k++) {
            const float cv = Store<T>::load1(cb + ch0 + fast_div(vidx(k, tid), p.hw_vec));
            float f[EPV];
            Store<T>::unpack(raw[k], f);
#pragma unroll
            for (int e = 0; e < EPV; e++) f[e] += cv;
            raw[k] = Store<T>::pack(f);
        }
    }
    if (!FULL) {  // registers of lanes past the end of a ragged slice hold zeros from here on
#pragma unroll
        for (int k = 0; k < K; k++) {
            const bool mine = have(k, tid);
#pragma unroll
            for (int i = 0; i < 4; i++) raw[k][i] = mine ? raw[k][i] : 0u;
        }
    }
    // per-vector channel affine.  Up to six vectors per lane: fetched into registers up front,
    // while the data is in flight.  More: the group's gamma and beta go to LDS once (they are
    // there after the barrier of the statistics) and the epilogue reads each vector's pair one
    // vector ahead, so a lane's registers hold little besides its packed slice.
    constexpr bool kPrefetchAffine = K <= kGnPrefetchAffineK;
    float ga[kPrefetchAffine ? K : 1], be[kPrefetchAffine ? K : 1];
    if (kPrefetchAffine) {
#pragma unroll
        for (int k = 0; k < K; k++) {
            const uint32_t c = ch0 + fast_div(vidx(k, tid), p.hw_vec);
            ga[kPrefetchAffine ? k : 0] = gamma[c];
            be[kPrefetchAffine ? k : 0] = beta[c];
        }
    } else {
        for (uint32_t c = tid; c < p.ch_per_group; c += nt) {  // ch_per_group <= kGnLdsChannels (host)
            aff[c] = make_float2(gamma[ch0 + c], beta[ch0 + c]);
        }
    }

    float slice_mean, slice_m2;
    gn_slice_stats<T, K, FULL>(raw, v_end - v_begin, red_a, red_b, red_c, slice_mean, slice_m2);

    float mean, rstd;
    uint32_t arrived_before = 0;
    if (SHARED || p.split == 1) {
        mean = slice_mean;
        rstd = __builtin_amdgcn_rsqf(slice_m2 * p.inv_count + p.eps);
    } else {
        // vector i of slice l as the statistics see it (input plus the optional addend)
        auto read = [&](uint32_t l, uint32_t i) {
            const uint32_t v = l * p.vec_per_slice + i;
            u32x4 r = xin[v];
            if (chunk != nullptr) {
                const T *cb = chunk + (size_t)(unit / p.groups) * (p.groups * p.ch_per_group);
                const float cv = Store<T>::load1(cb + ch0 + fast_div(v, p.hw_vec));
                float f[EPV];
                Store<T>::unpack(r, f);
#pragma unroll
                for (int e = 0; e < EPV; e++) f[e] += cv;
                r = Store<T>::pack(f);
            }
            return r;
        };
        gn_exchange<T>(scratch, p, unit, slice, epoch, slice_mean, slice_m2, stats, read);
        mean = stats[0];
        rstd = stats[1];
        if (tid == 0) arrived_before = gn_exchange_arrive(scratch, unit);
    }

    // ---- normalise from registers, per-channel affine, optional SiLU.  When the unit's mean is
    // within four standard deviations of zero it is folded into the offset,
    // y = fma(x, a, beta - mean a) (one operation per element, error a few 1e-7 at most);
    // otherwise y = fma(x - mean, a, beta), which stays exact for |mean| >> sigma.
    auto epilogue = [&](auto fold_tag) {
        constexpr bool kFold = decltype(fold_tag)::value;
        float g_next = 0.0f, b_next = 0.0f;
        if (!kPrefetchAffine) {
            const uint32_t c = fast_div(vidx(0, lane_again()), p.hw_vec);
            const float2 gb = aff[c];  // one 8-byte LDS read
            g_next = gb.x;
            b_next = gb.y;
        }
#pragma unroll
        for (int k = 0; k < K; k++) {
            float g_k, b_k;
            if (kPrefetchAffine) {
                g_k = ga[kPrefetchAffine ? k : 0];
                b_k = be[kPrefetchAffine ? k : 0];
            } else {
                g_k = g_next;
                b_k = b_next;
                if (k + 1 < K) {  // the next vector's pair: its LDS latency passes under this vector's work
                    const uint32_t c = fast_div(vidx(k + 1, lane_again()), p.hw_vec);
                    const float2 gb = aff[c];
                    g_next = gb.x;
                    b_next = gb.y;
                }
            }
            // several writers per unit: this one normalises and stores the vectors of its part
            // only; a wavefront is inside a part or outside it as a whole
            if (SHARED) {  // (decided per wavefront: a scalar branch)
                const uint32_t first = __builtin_amdgcn_readfirstlane(vidx(k, lane_again()));
                if (first - part * p.part_vecs >= p.part_vecs) continue;
            }
            const float a = rstd * g_k;
            const float b_fold = fmaf(-mean, a, b_k);
            float f[EPV];
            forget(raw[k]);  // unpack here, one vector at a time
            Store<T>::unpack(raw[k], f);
#pragma unroll
            for (int e = 0; e < EPV; e++) {
                const float t = kFold ? fmaf(f[e], a, b_fold) : fmaf(f[e] - mean, a, b_k);
                f[e] = SILU ? silu_f(t) : t;
            }
            const u32x4 packed = Store<T>::pack(f);
            const uint32_t t = lane_again();
            if (have(k, t)) store_stream(at(yout, k, t), packed);
            // the scheduler must not start unpacking the next vectors before this one is stored:
            // eight elements are enough independent work, and the slice stays packed until used
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    if (mean * mean * (rstd * rstd) <= kGnFoldMean)  // uniform over the workgroup
        epilogue(std::true_type{});
    else
        epilogue(std::false_type{});
    if (!SHARED && p.split > 1 && tid == 0) gn_exchange_close(scratch, p, unit, epoch, arrived_before);
}

// Up to five vectors per lane (four for float storage) the kernel fits 64 registers: eight
// wavefronts per SIMD, so two 1024-lane workgroups share a CU and one loads while the other
// computes (what large batches need).
template <typename T, int K, bool SILU, bool SHARED>
__global__ __launch_bounds__(kGnMaxThreads, (K <= (sizeof(T) == 2 ? 5 : 4) ? 8 : 4)) void gn_slice_kernel(
    const T *x, const T *chunk, T *y, const float *__restrict__ gamma,
    const float *__restrict__ beta, GnScratch scratch, GnParams p) {
    __shared__ float red_a[kGnMaxThreads / kWave];
    __shared__ float red_b[kGnMaxThreads / kWave];
    __shared__ float red_c[kGnMaxThreads / kWave];
    __shared__ float stats[2];
    __shared__ float2 aff[K <= kGnPrefetchAffineK ? 1 : kGnLdsChannels];  // (gamma, beta) of the group's channels
    uint32_t unit, slice, part;
    if (SHARED) {  // whole units, `writers` workgroups each
        const uint32_t j = blockIdx.x >> p.xcd_shift;
        part = j & (p.writers - 1);
        unit = ((j >> p.writers_shift) << p.xcd_shift) + (blockIdx.x & ((1u << p.xcd_shift) - 1u));
        slice = 0;
    } else {
        unit = blockIdx.x >> p.split_shift;
        slice = blockIdx.x & (p.split - 1);
        part = 0;
    }
    const uint32_t v_begin = slice * p.vec_per_slice;
    const uint32_t v_end = min(p.vec_per_unit, v_begin + p.vec_per_slice);
    // uniform over the workgroup; the largest K is only launched on slices it fits exactly
    if (K == kGnMaxK || v_end - v_begin == K * blockDim.x)
        gn_body<T, K, SILU, true, SHARED>(x, chunk, y, gamma, beta, scratch, p, unit, slice, part, v_begin, v_end,
                                          red_a, red_b, red_c, stats, aff);
    else
        gn_body<T, K, SILU, false, SHARED>(x, chunk, y, gamma, beta, scratch, p, unit, slice, part, v_begin, v_end,
                                           red_a, red_b, red_c, stats, aff);
}

// Any shape or alignment: one workgroup per unit, three passes over global memory with
// scalar accesses (the second and third pass hit in cache for UNet-sized units).
template <typename T, bool SILU>
__global__ __launch_bounds__(kGenericThreads) void gn_generic_kernel(
    const T *x, const T *chunk, T *y, const float *__restrict__ gamma,
    const float *__restrict__ beta, uint32_t unit_size, uint32_t hw, uint32_t groups,
    uint32_t ch_per_group, float eps) {
    __shared__ float red_a[kGenericThreads / kWave];
    __shared__ float red_b[kGenericThreads / kWave];
    const uint32_t unit = blockIdx.x;
    const T *xin = x + (size_t)unit * unit_size;
    T *yout = y + (size_t)unit * unit_size;
    const uint32_t ch0 = (unit % groups) * ch_per_group;
    const T *cb = chunk ? chunk + (size_t)(unit / groups) * (groups * ch_per_group) + ch0 : nullptr;
    // element i of the unit, with the optional addend, rounded to the storage type
    auto value = [&](uint32_t i) {
        float v = Store<T>::load1(xin + i);
        if (cb) v = round_to_storage<T>(v + Store<T>::load1(cb + i / hw));
        return v;
    };
    float s = 0.0f;
    for (uint32_t i = threadIdx.x; i < unit_size; i += kGenericThreads) s += value(i);
    const float mean = block_sum_rt(s, red_a) / (float)unit_size;
    float q = 0.0f;
    for (uint32_t i = threadIdx.x; i < unit_size; i += kGenericThreads) {
        const float d = value(i) - mean;
        q = fmaf(d, d, q);
    }
    const float rstd = 1.0f / sqrtf(block_sum_rt(q, red_b) / (float)unit_size + eps);
    // every lane re-reads only elements it writes itself, so y may alias x
    for (uint32_t i = threadIdx.x; i < unit_size; i += kGenericThreads) {
        const uint32_t c = ch0 + i / hw;
        const float t = fmaf(value(i) - mean, rstd * gamma[c], beta[c]);
        Store<T>::store1(yout + i, SILU ? silu_f(t) : t);
    }
}

// ---------------------------------------------------------------------------
// GroupNorm with a token-major store: y[b, p, c] = GroupNorm(x)[b, c, p].
// Replaces GroupNorm followed by the (0, 2, 1) permute that turns NCHW into tokens.
// A slice is all channels of the group over a range of positions, so that for each position
// the slice owns one contiguous run of ch_per_group outputs; normalised values go through
// LDS ([channel][position], 16-byte padded pitch) and leave as 4-byte stores that walk those
// runs.  Statistics and the exchange between slices are those of gn_slice_kernel.
// ---------------------------------------------------------------------------
struct GnTokParams {
    GnParams base;        // vec_per_slice = ch_per_group * pos_vecs.d ; vec_per_unit = that * split
    FastDiv pos_vecs;     // position vectors per slice (hw_vec / split)
    FastDiv row_dwords;   // 4-byte words per output run: ch_per_group * sizeof(T) / 4
    uint32_t hw;          // positions per sample
    uint32_t channels;
    uint32_t pitch;       // LDS elements between channels: positions per slice + 16 bytes
    FastDiv combos;       // batch * split: (sample, slice) pairs, the fastest part of the block id
    FastDiv part_len;     // SHARED: vectors of one part, ch_per_group * pos_vecs.d (a multiple of 64)
};

// SHARED: `writers` workgroups per whole unit (output apart from the input by construction).  Each
// loads and reduces the whole unit, enumerated part by part (a part = all channels over a range of
// positions, what a slice is above), and normalises, transposes and stores its own part; nothing
// is exchanged.  The writers of a unit have block ids one XCD count apart (one XCD: their loads meet in
// its L2).
template <typename T, int K, bool SHARED>
__global__ __launch_bounds__(kGnMaxThreads) void gn_tokens_kernel(
    const T *__restrict__ x, T *__restrict__ y, const float *__restrict__ gamma,
    const float *__restrict__ beta, GnScratch scratch, GnTokParams q) {
    constexpr int EPV = Store<T>::EPV;
    extern __shared__ u32x4 lds_vec[];
    __shared__ float red_a[kGnMaxThreads / kWave];
    __shared__ float red_b[kGnMaxThreads / kWave];
    __shared__ float red_c[kGnMaxThreads / kWave];
    __shared__ float stats[2];
    const GnParams &p = q.base;
    const uint32_t tid = threadIdx.x;
    const uint32_t nt = blockDim.x;
    // block id = group * (batch * split) + sample * split + slice: the workgroups that write
    // pieces of the same output lines (all groups of one sample and position range) have ids
    // that differ by multiples of batch * split, so with workgroups dealt round-robin to the
    // 8 XCDs they meet in one L2 when that product is a multiple of 8 (batch 2 x 4 slices);
    // the slices of a unit stay adjacent
    uint32_t unit, slice;  // SHARED: `slice` is the part this workgroup stores
    if (SHARED) {
        const uint32_t j = blockIdx.x >> p.xcd_shift;
        slice = j & (p.writers - 1);
        unit = ((j >> p.writers_shift) << p.xcd_shift) + (blockIdx.x & ((1u << p.xcd_shift) - 1u));
    } else {
        const uint32_t group = fast_div(blockIdx.x, q.combos);
        const uint32_t combo = blockIdx.x - group * q.combos.d;
        unit = (combo >> p.split_shift) * p.groups + group;
        slice = combo & (p.split - 1);
    }
    const uint32_t nvec = SHARED ? p.vec_per_unit : p.vec_per_slice;  // vectors this workgroup holds
    const uint32_t pvs = q.pos_vecs.d;
    const u32x4 *xin = reinterpret_cast<const u32x4 *>(x) + (size_t)unit * p.vec_per_unit;

    uint32_t epoch = 0;
    if (!SHARED && p.split > 1 && tid == 0)
        epoch = __hip_atomic_load(scratch.epoch + unit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // lane-local vector -> (part, channel of the group, position vector of the part / slice)
    u32x4 raw[K];
    uint32_t cl[K], pv[K];
#pragma unroll
    for (int k = 0; k < K; k++) {
        uint32_t vl = min(k * nt + tid, nvec - 1);  // ragged tail re-reads the last vector
        uint32_t part_of = slice;
        if (SHARED) {
            part_of = fast_div(vl, q.part_len);
            vl -= part_of * q.part_len.d;
        }
        cl[k] = fast_div(vl, q.pos_vecs);
        pv[k] = vl - cl[k] * pvs;
        raw[k] = load_stream(xin + (size_t)cl[k] * p.hw_vec.d + part_of * pvs + pv[k]);
        const bool have = k * nt + tid < nvec;  // lanes past the end hold zeros (the statistics rely on it)
#pragma unroll
        for (int i = 0; i < 4; i++) raw[k][i] = have ? raw[k][i] : 0u;
    }
    const uint32_t ch0 = (unit % p.groups) * p.ch_per_group;

    float slice_mean, slice_m2;
    gn_slice_stats<T, K, false>(raw, nvec, red_a, red_b, red_c, slice_mean, slice_m2);

    float mean, rstd;
    if (SHARED || p.split == 1) {
        mean = slice_mean;
        rstd = __builtin_amdgcn_rsqf(slice_m2 * p.inv_count + p.eps);
    } else {
        // vector i of slice l: channel i / pos_vecs of the group, position vector i % pos_vecs
        auto read = [&](uint32_t l, uint32_t i) {
            const uint32_t c = fast_div(i, q.pos_vecs);
            return xin[(size_t)c * p.hw_vec.d + l * pvs + (i - c * pvs)];
        };
        gn_exchange<T>(scratch, p, unit, slice, epoch, slice_mean, slice_m2, stats, read);
        mean = stats[0];
        rstd = stats[1];
    }

    // ---- normalise into LDS as [channel][position]
    T *lds = reinterpret_cast<T *>(lds_vec);
#pragma unroll
    for (int k = 0; k < K; k++) {
        if (SHARED) {  // a wavefront lies inside one part (part_len is a multiple of 64): a scalar branch
            const uint32_t first = __builtin_amdgcn_readfirstlane(min(k * nt + tid, nvec - 1));
            if (first - slice * q.part_len.d >= q.part_len.d) continue;
        }
        if (k * nt + tid < nvec) {
            const float a = rstd * gamma[ch0 + cl[k]];
            const float b = beta[ch0 + cl[k]];
            float f[EPV];
            Store<T>::unpack(raw[k], f);
#pragma unroll
            for (int e = 0; e < EPV; e++) f[e] = fmaf(f[e] - mean, a, b);
            *reinterpret_cast<u32x4 *>(lds + (size_t)cl[k] * q.pitch + pv[k] * EPV) = Store<T>::pack(f);
        }
    }
    __syncthreads();
    // the slice counts itself done here, behind the last barrier: nothing waits for the answer
    uint32_t arrived_before = 0;
    if (!SHARED && p.split > 1 && tid == 0) arrived_before = gn_exchange_arrive(scratch, unit);

    // ---- token-major store: for each position of the slice one run of ch_per_group values
    const uint32_t rows = pvs * EPV;                         // positions in the slice
    const uint32_t words = rows * q.row_dwords.d;            // 4-byte words to write
    const uint32_t sample = unit / p.groups;
    const size_t first = ((size_t)sample * q.hw + (size_t)slice * rows) * q.channels + ch0;
    uint32_t *out = reinterpret_cast<uint32_t *>(y + first);
    const uint32_t row_stride = q.channels * sizeof(T) / 4;  // words between positions
    for (uint32_t i = tid; i < words; i += nt) {
        const uint32_t r = fast_div(i, q.row_dwords);
        const uint32_t c = i - r * q.row_dwords.d;
        uint32_t w;
        if (sizeof(T) == 2) {
            const uint16_t lo = reinterpret_cast<const uint16_t *>(lds)[(2 * c) * q.pitch + r];
            const uint16_t hi = reinterpret_cast<const uint16_t *>(lds)[(2 * c + 1) * q.pitch + r];
            w = (uint32_t)lo | ((uint32_t)hi << 16);
        } else {
            w = reinterpret_cast<const uint32_t *>(lds)[c * q.pitch + r];
        }
        out[(size_t)r * row_stride + c] = w;
    }
    if (!SHARED && p.split > 1 && tid == 0) gn_exchange_close(scratch, p, unit, epoch, arrived_before);
}

// Any shape: one workgroup per unit, three passes, element-wise scattered stores.
template <typename T>
__global__ __launch_bounds__(kGenericThreads) void gn_tokens_generic_kernel(
    const T *__restrict__ x, T *__restrict__ y, const float *__restrict__ gamma,
    const float *__restrict__ beta, uint32_t unit_size, uint32_t hw, uint32_t groups,
    uint32_t ch_per_group, float eps) {
    __shared__ float red_a[kGenericThreads / kWave];
    __shared__ float red_b[kGenericThreads / kWave];
    const uint32_t unit = blockIdx.x;
    const T *xin = x + (size_t)unit * unit_size;
    float s = 0.0f;
    for (uint32_t i = threadIdx.x; i < unit_size; i += kGenericThreads) s += Store<T>::load1(xin + i);
    const float mean = block_sum_rt(s, red_a) / (float)unit_size;
    float m2 = 0.0f;
    for (uint32_t i = threadIdx.x; i < unit_size; i += kGenericThreads) {
        const float d = Store<T>::load1(xin + i) - mean;
        m2 = fmaf(d, d, m2);
    }
    const float rstd = 1.0f / sqrtf(block_sum_rt(m2, red_b) / (float)unit_size + eps);
    const uint32_t ch0 = (unit % groups) * ch_per_group;
    const uint32_t channels = groups * ch_per_group;
    T *yout = y + (size_t)(unit / groups) * hw * channels;
    for (uint32_t i = threadIdx.x; i < unit_size; i += kGenericThreads) {
        const uint32_t c = ch0 + i / hw, pos = i % hw;
        const float t = fmaf(Store<T>::load1(xin + i) - mean, rstd * gamma[c], beta[c]);
        Store<T>::store1(yout + (size_t)pos * channels + c, t);
    }
}

// ---------------------------------------------------------------------------
// Host: launches (the plan comes from gn_plan.hip)
// ---------------------------------------------------------------------------
// log2 of the distance between the block ids of a unit's writers: the XCD count when the
// workgroups of a launch are dealt to a power-of-two number of XCDs in turn and the units come
// in whole rows of that many (the writers then share an XCD), else 0 (adjacent ids).
inline uint32_t gn_xcd_shift(const Chip &chip, bool shared, size_t units) {
    if (!shared || chip.xcds <= 1 || (chip.xcds & (chip.xcds - 1)) != 0 || units % chip.xcds != 0) return 0;
    return (uint32_t)__builtin_ctz(chip.xcds);
}

template <typename T, int K>
void gn_launch_k(bool silu, bool shared, uint32_t blocks, uint32_t threads, hipStream_t stream, const T *x,
                 const T *chunk, T *y, const float *gamma, const float *beta, const GnScratch &sc,
                 const GnParams &p) {
    if (K <= kGnSharedMaxK && shared) {
        constexpr int KS = K <= kGnSharedMaxK ? K : 1;  // (larger K never get here: no such instances)
        if (silu)
            launch((gn_slice_kernel<T, KS, true, true>), dim3(blocks), dim3(threads), 0, stream, x,
                               chunk, y, gamma, beta, sc, p);
        else
            launch((gn_slice_kernel<T, KS, false, true>), dim3(blocks), dim3(threads), 0, stream,
                               x, chunk, y, gamma, beta, sc, p);
    } else if (silu) {
        launch((gn_slice_kernel<T, K, true, false>), dim3(blocks), dim3(threads), 0, stream, x,
                           chunk, y, gamma, beta, sc, p);
    } else {
        launch((gn_slice_kernel<T, K, false, false>), dim3(blocks), dim3(threads), 0, stream,
                           x, chunk, y, gamma, beta, sc, p);
    }
}

template <typename T>
int gn_generic(bool silu, const T *x, const T *chunk, T *y, const float *gamma, const float *beta,
               size_t units, size_t unit_size, size_t hw, size_t groups, size_t cpg, float eps,
               hipStream_t stream) {
    launch((silu ? gn_generic_kernel<T, true> : gn_generic_kernel<T, false>),
                       dim3((uint32_t)units), dim3(kGenericThreads), 0, stream, x, chunk, y, gamma, beta,
                       (uint32_t)unit_size, (uint32_t)hw, (uint32_t)groups, (uint32_t)cpg, eps);
    return launch_status();
}

}  // namespace

template <typename T>
int gn_dispatch(const void *xv, const void *chunkv, void *yv, const float *gamma, const float *beta,
                size_t batch, size_t channels, size_t hw, size_t groups, float eps, bool silu,
                const GnScratch *fixed, hipStream_t stream) {
    constexpr int EPV = Store<T>::EPV;
    const int tune_spin = g_tuning.gn_spin_limit.load(std::memory_order_relaxed);
    const T *x = static_cast<const T *>(xv);
    const T *chunk = static_cast<const T *>(chunkv);
    T *y = static_cast<T *>(yv);
    const size_t cpg = channels / groups;
    const size_t unit_size = cpg * hw;
    const size_t units = batch * groups;
    if (units == 0 || unit_size == 0) return MSD_OK;
    if (units > 0x7FFFFFFFull || unit_size > 0x7FFFFFFFull) return MSD_ERR_INVALID_VALUE;
    if (fixed != nullptr && units > fixed->units) return MSD_ERR_SCRATCH_LIMIT;
    // several workgroups may share a unit only if none of them can store into what another still
    // loads: the output must lie apart from the input
    const char *xb = reinterpret_cast<const char *>(x), *yb = reinterpret_cast<const char *>(y);
    const size_t bytes = units * unit_size * sizeof(T);
    const bool apart = xb + bytes <= yb || yb + bytes <= xb;
    const GnDecision d = gn_decide(sizeof(T), batch, channels, hw, groups, aligned16(x) && aligned16(y),
                                   fixed != nullptr ? fixed->units : kGnMaxUnits, apart);
    if (d.split == 0)
        return gn_generic<T>(silu, x, chunk, y, gamma, beta, units, unit_size, hw, groups, cpg, eps, stream);

    const uint32_t split = d.split;
    GnParams p;
    p.vec_per_unit = (uint32_t)(unit_size / EPV);
    p.vec_per_slice = d.vec_per_slice;
    p.split = split;
    p.split_shift = (uint32_t)__builtin_ctz(split);
    p.groups = (uint32_t)groups;
    p.ch_per_group = (uint32_t)cpg;
    p.hw_vec = make_fast_div((uint32_t)(hw / EPV));
    p.eps = eps;
    p.inv_count = 1.0f / (float)unit_size;
    p.spin_limit = tune_spin > 0 ? (uint32_t)tune_spin : kGnSpinLimit;
    const bool shared = d.writers > 1;
    p.writers = d.writers;
    p.writers_shift = (uint32_t)__builtin_ctz(d.writers);
    p.part_vecs = (uint32_t)((((p.vec_per_unit + d.writers - 1) / d.writers + kWave - 1) / kWave) * kWave);
    p.xcd_shift = gn_xcd_shift(chip_info(), shared, units);

    GnScratch sc{nullptr, nullptr, nullptr, nullptr, nullptr, 0};
    if (fixed != nullptr) {
        sc = *fixed;
    } else if (split > 1) {
        const hipError_t err = get_scratch(stream, &sc);
        if (err != hipSuccess) return (int)err;
    }
    const uint32_t blocks = (uint32_t)(units * split * d.writers);
    const uint32_t threads = d.threads;
    switch (d.k) {
        case 1: gn_launch_k<T, 1>(silu, shared, blocks, threads, stream, x, chunk, y, gamma, beta, sc, p); break;
        case 2: gn_launch_k<T, 2>(silu, shared, blocks, threads, stream, x, chunk, y, gamma, beta, sc, p); break;
        case 3: gn_launch_k<T, 3>(silu, shared, blocks, threads, stream, x, chunk, y, gamma, beta, sc, p); break;
        case 4: gn_launch_k<T, 4>(silu, shared, blocks, threads, stream, x, chunk, y, gamma, beta, sc, p); break;
        case 5: gn_launch_k<T, 5>(silu, shared, blocks, threads, stream, x, chunk, y, gamma, beta, sc, p); break;
        case 6: gn_launch_k<T, 6>(silu, shared, blocks, threads, stream, x, chunk, y, gamma, beta, sc, p); break;
        case 8: gn_launch_k<T, 8>(silu, shared, blocks, threads, stream, x, chunk, y, gamma, beta, sc, p); break;
        case 10: gn_launch_k<T, 10>(silu, shared, blocks, threads, stream, x, chunk, y, gamma, beta, sc, p); break;
        case 12: gn_launch_k<T, 12>(silu, shared, blocks, threads, stream, x, chunk, y, gamma, beta, sc, p); break;
        case 16: gn_launch_k<T, 16>(silu, shared, blocks, threads, stream, x, chunk, y, gamma, beta, sc, p); break;
        case 20: gn_launch_k<T, 20>(silu, shared, blocks, threads, stream, x, chunk, y, gamma, beta, sc, p); break;
        default: return MSD_ERR_INVALID_VALUE;  // not a K the kernels are built for: a planning error
    }
    return launch_status();
}

template int gn_dispatch<float>(const void *, const void *, void *, const float *, const float *,
                                size_t, size_t, size_t, size_t, float, bool, const GnScratch *, hipStream_t);
template int gn_dispatch<__half>(const void *, const void *, void *, const float *, const float *,
                                 size_t, size_t, size_t, size_t, float, bool, const GnScratch *, hipStream_t);

namespace {

template <typename T, int K>
void gn_tokens_launch(bool shared, uint32_t blocks, uint32_t threads, size_t lds_bytes, hipStream_t stream,
                      const T *x, T *y, const float *gamma, const float *beta, const GnScratch &sc,
                      const GnTokParams &q) {
    if (K <= kGnSharedMaxK && shared) {
        constexpr int KS = K <= kGnSharedMaxK ? K : 1;  // (no instances with several writers beyond that)
        launch((gn_tokens_kernel<T, KS, true>), dim3(blocks), dim3(threads), lds_bytes, stream, x, y,
                           gamma, beta, sc, q);
    } else {
        launch((gn_tokens_kernel<T, K, false>), dim3(blocks), dim3(threads), lds_bytes, stream, x, y,
                           gamma, beta, sc, q);
    }
}

}  // namespace

template <typename T>
int gn_tokens_dispatch(const void *xv, void *yv, const float *gamma, const float *beta, size_t batch,
                       size_t channels, size_t hw, size_t groups, float eps, hipStream_t stream) {
    constexpr int EPV = Store<T>::EPV;
    constexpr uint32_t kMaxK = sizeof(T) == 4 ? 10 : kGnMaxRaggedK;
    constexpr size_t kMaxLds = 60 * 1024;
    const T *x = static_cast<const T *>(xv);
    T *y = static_cast<T *>(yv);
    const size_t cpg = channels / groups;
    const size_t unit_size = cpg * hw;
    const size_t units = batch * groups;
    if (units == 0 || unit_size == 0) return MSD_OK;
    if (units > 0x7FFFFFFFull || unit_size > 0x7FFFFFFFull) return MSD_ERR_INVALID_VALUE;
    auto generic = [&]() {
        launch((gn_tokens_generic_kernel<T>), dim3((uint32_t)units), dim3(kGenericThreads), 0,
                           stream, x, y, gamma, beta, (uint32_t)unit_size, (uint32_t)hw, (uint32_t)groups,
                           (uint32_t)cpg, eps);
        return launch_status();
    };
    const bool vector_ok = aligned16(x) && (reinterpret_cast<uintptr_t>(y) & 3u) == 0 && hw % EPV == 0 &&
                           (cpg * sizeof(T)) % 4 == 0 && (channels * sizeof(T)) % 4 == 0;
    if (!vector_ok) return generic();
    const size_t hw_vec = hw / EPV;
    // slices cut the positions: the split must divide them, fit the registers and the LDS.
    // Cut earlier than gn_dispatch does: the block layout puts the workgroups that write pieces
    // of the same output lines on one XCD when batch * split is a multiple of the XCD count, which
    // is worth more than the exchange costs from 16 Ki elements on.  With half a workgroup per CU
    // or more, units stay whole or (exactly half) go in two; four slices otherwise, eight when
    // even that leaves a quarter of the chip idle and a slice keeps 4 Ki elements.
    const Chip chip = chip_info();
    uint32_t want = 1;
    if (unit_size > 16384) {
        want = units * 2 > chip.cus ? 1 : units * 2 == chip.cus ? 2 : 4;
        if (units * 16 < 3 * (size_t)chip.cus && unit_size >= 32768) want = 8;
    }
    const int tune_split = g_tuning.gn_split.load(std::memory_order_relaxed);
    const int tune_spin = g_tuning.gn_spin_limit.load(std::memory_order_relaxed);
    if (tune_split > 0) want = (uint32_t)tune_split;
    uint32_t split = 0;
    for (uint32_t s = 1; s <= kGnMaxSplit; s *= 2) {
        if (hw_vec % s != 0) break;
        const size_t nvec = cpg * (hw_vec / s);
        const size_t lds = cpg * (hw / s + 16 / sizeof(T)) * sizeof(T);
        if (nvec > (size_t)kGnMaxThreads * kMaxK || lds > kMaxLds) continue;
        split = s;
        if (s >= want) break;
    }
    // Several writers per whole unit instead of slices with an exchange (see gn_auto_writers): the
    // parts cut the positions like slices do, must divide them, hold whole wavefronts' vectors
    // and fit the LDS; the whole unit must fit the registers of one workgroup.
    const int tune_writers = g_tuning.gn_writers.load(std::memory_order_relaxed);
    uint32_t writers = 1;
    const size_t vec_per_unit = cpg * hw_vec;
    const char *xb = reinterpret_cast<const char *>(x), *yb = reinterpret_cast<const char *>(y);
    const size_t bytes = units * unit_size * sizeof(T);
    const bool apart = xb + bytes <= yb || yb + bytes <= xb;
    if (apart && tune_split <= 1 && tune_writers != 1 && vec_per_unit <= (size_t)kGnMaxThreads * kGnSharedMaxK) {
        uint32_t w = tune_writers > 1 ? (uint32_t)tune_writers : gn_auto_writers(chip, sizeof(T), units, vec_per_unit);
        // Here the limit is lower than for the channel-major store: the slices of a cut unit
        // also keep the writers of an output line on one XCD, which the writers of a unit give
        // up.  Measured, batch 2 fp16, several writers against slices: 1280 channels at 16 x 16
        // 4.03 against 4.64 us, 640 at 32 x 32 5.79 against 6.11, 320 at 64 x 64 9.14 against
        // 7.90; batch 4 (two writers): 4.72 against 5.13, 7.45 against 7.07.
        if (tune_writers <= 1 && unit_size > (w >= 4 ? 20480u : 10240u)) w = 1;
        for (; w > 1; w /= 2) {
            if (hw_vec % w != 0) continue;
            const size_t part_len = cpg * (hw_vec / w);
            const size_t lds = cpg * (hw / w + 16 / sizeof(T)) * sizeof(T);
            if (part_len % kWave == 0 && lds <= kMaxLds) break;
        }
        writers = (w < 1 || units * w > 0x7FFFFFFFull) ? 1 : w;  // (the grid is units * writers blocks)
        if (writers > 1 &&
            gn_threads_for(chip, sizeof(T), (uint32_t)vec_per_unit, 1, units * writers, kGnSharedMaxK, true, true).k == 0)
            writers = 1;  // (the whole unit does not fit one workgroup's registers: slices as below)
    }
    const bool shared = writers > 1;
    if (!shared && (split == 0 || (split > 1 && units > kGnMaxUnits))) return generic();
    if (shared) split = 1;

    GnTokParams q;
    const size_t pvs = hw_vec / (shared ? writers : split);  // position vectors of a part / slice
    const size_t nvec = cpg * pvs;
    q.base.vec_per_unit = (uint32_t)vec_per_unit;
    q.base.vec_per_slice = (uint32_t)nvec;
    q.base.split = split;
    q.base.split_shift = (uint32_t)__builtin_ctz(split);
    q.base.writers = writers;
    q.base.writers_shift = (uint32_t)__builtin_ctz(writers);
    q.base.part_vecs = (uint32_t)nvec;
    q.base.xcd_shift = gn_xcd_shift(chip, shared, units);
    q.base.groups = (uint32_t)groups;
    q.base.ch_per_group = (uint32_t)cpg;
    q.base.hw_vec = make_fast_div((uint32_t)hw_vec);
    q.base.eps = eps;
    q.base.inv_count = 1.0f / (float)unit_size;
    q.base.spin_limit = tune_spin > 0 ? (uint32_t)tune_spin : kGnSpinLimit;
    q.pos_vecs = make_fast_div((uint32_t)pvs);
    q.row_dwords = make_fast_div((uint32_t)(cpg * sizeof(T) / 4));
    q.hw = (uint32_t)hw;
    q.channels = (uint32_t)channels;
    q.pitch = (uint32_t)(pvs * EPV + 16 / sizeof(T));
    q.combos = make_fast_div((uint32_t)(batch * split));
    q.part_len = make_fast_div((uint32_t)nvec);
    const size_t lds_bytes = cpg * q.pitch * sizeof(T);
    // a workgroup holds its slice, or with several writers the whole unit
    const GnThreads pl = shared ? gn_threads_for(chip, sizeof(T), (uint32_t)vec_per_unit, 1, units * writers, kGnSharedMaxK,
                                                 true, true)
                                : gn_threads_for(chip, sizeof(T), (uint32_t)nvec, split, units * split, kMaxK, false, false);
    if (pl.k == 0) return generic();
    GnScratch sc{nullptr, nullptr, nullptr, nullptr, nullptr, 0};
    if (!shared && split > 1) {
        const hipError_t err = get_scratch(stream, &sc);
        if (err != hipSuccess) return (int)err;
    }
    const uint32_t blocks = (uint32_t)(units * (shared ? writers : split));
    const uint32_t threads = pl.threads;
    switch (pl.k) {
        case 1: gn_tokens_launch<T, 1>(shared, blocks, threads, lds_bytes, stream, x, y, gamma, beta, sc, q); break;
        case 2: gn_tokens_launch<T, 2>(shared, blocks, threads, lds_bytes, stream, x, y, gamma, beta, sc, q); break;
        case 3: gn_tokens_launch<T, 3>(shared, blocks, threads, lds_bytes, stream, x, y, gamma, beta, sc, q); break;
        case 4: gn_tokens_launch<T, 4>(shared, blocks, threads, lds_bytes, stream, x, y, gamma, beta, sc, q); break;
        case 5: gn_tokens_launch<T, 5>(shared, blocks, threads, lds_bytes, stream, x, y, gamma, beta, sc, q); break;
        case 6: gn_tokens_launch<T, 6>(shared, blocks, threads, lds_bytes, stream, x, y, gamma, beta, sc, q); break;
        case 8: gn_tokens_launch<T, 8>(shared, blocks, threads, lds_bytes, stream, x, y, gamma, beta, sc, q); break;
        case 10: gn_tokens_launch<T, 10>(shared, blocks, threads, lds_bytes, stream, x, y, gamma, beta, sc, q); break;
        case 12: gn_tokens_launch<T, 12>(shared, blocks, threads, lds_bytes, stream, x, y, gamma, beta, sc, q); break;
        default: gn_tokens_launch<T, 16>(shared, blocks, threads, lds_bytes, stream, x, y, gamma, beta, sc, q); break;
    }
    return launch_status();
}

template int gn_tokens_dispatch<float>(const void *, void *, const float *, const float *, size_t, size_t,
                                       size_t, size_t, float, hipStream_t);
template int gn_tokens_dispatch<__half>(const void *, void *, const float *, const float *, size_t, size_t,
                                        size_t, size_t, float, hipStream_t);

}  // namespace msd
