// Device-side building blocks shared by the gfx950 kernels: 16-byte packed
// access for float / half storage, DPP reductions for 64-wide wavefronts,
// activation math, and a multiply-shift replacement for integer division.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace msd {

constexpr int kWave = 64;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------------------
// Storage traits: one 16-byte vector holds EPV elements.
// ---------------------------------------------------------------------------
template <typename T>
struct Store;

template <>
struct Store<float> {
    static constexpr int EPV = 4;
    static __device__ __forceinline__ void unpack(const u32x4 &v, float *f) {
#pragma unroll
        for (int i = 0; i < 4; i++) f[i] = __uint_as_float(v[i]);
    }
    static __device__ __forceinline__ u32x4 pack(const float *f) {
        u32x4 v;
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] = __float_as_uint(f[i]);
        return v;
    }
    static __device__ __forceinline__ float load1(const float *p) { return *p; }
    static __device__ __forceinline__ void store1(float *p, float v) { *p = v; }
};

template <>
struct Store<__half> {
    static constexpr int EPV = 8;
    static __device__ __forceinline__ void unpack(const u32x4 &v, float *f) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t w = v[i];
            const __half2 h = *reinterpret_cast<const __half2 *>(&w);
            const float2 t = __half22float2(h);
            f[2 * i] = t.x;
            f[2 * i + 1] = t.y;
        }
    }
    static __device__ __forceinline__ u32x4 pack(const float *f) {
        u32x4 v;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const __half2 h = __floats2half2_rn(f[2 * i], f[2 * i + 1]);  // round-to-nearest-even
            v[i] = *reinterpret_cast<const uint32_t *>(&h);
        }
        return v;
    }
    static __device__ __forceinline__ float load1(const __half *p) { return __half2float(*p); }
    static __device__ __forceinline__ void store1(__half *p, float v) { *p = __float2half_rn(v); }
};

// v as the storage type would hold it (identity for float, round-to-nearest-even for half)
template <typename T>
__device__ __forceinline__ float round_to_storage(float v);
template <>
__device__ __forceinline__ float round_to_storage<float>(float v) {
    return v;
}
template <>
__device__ __forceinline__ float round_to_storage<__half>(float v) {
    return __half2float(__float2half_rn(v));
}

// Streaming (read-once / write-once) 16-byte access.
__device__ __forceinline__ u32x4 load_stream(const u32x4 *p) {
    return __builtin_nontemporal_load(p);
}
__device__ __forceinline__ void store_stream(u32x4 *p, const u32x4 &v) {
    __builtin_nontemporal_store(v, p);
}

// Makes the compiler forget what it knows about a packed vector held in registers, so
// that conversions of it are redone where they are used instead of being kept live
// (unpacked copies of a register-resident slice would not fit the register file).
__device__ __forceinline__ void forget(u32x4 &v) {
    uint32_t a = v[0], b = v[1], c = v[2], d = v[3];
    asm volatile("" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
    v = u32x4{a, b, c, d};
}

// ---------------------------------------------------------------------------
// Division by a launch-time constant d (n < 2^31): q = umulhi(n, mul) >> shift.
// mul = ceil(2^(31+L) / d), shift = L-1 with L = ceil(log2 d), d >= 2; d == 1 is
// flagged with mul == 0.  Exact for every n < 2^31 (Granlund-Montgomery).
// ---------------------------------------------------------------------------
struct FastDiv {
    uint32_t mul;
    uint32_t shift;
    uint32_t d;
};

// Host side: the constants for divisor d.
inline FastDiv make_fast_div(uint32_t d) {
    FastDiv fd{0u, 0u, d};
    if (d <= 1) return fd;
    uint32_t L = 0;
    while ((1ull << L) < d) L++;
    fd.mul = (uint32_t)(((1ull << (31 + L)) + d - 1) / d);
    fd.shift = L - 1;
    return fd;
}

__device__ __forceinline__ uint32_t fast_div(uint32_t n, const FastDiv &fd) {
    const uint32_t q = __umulhi(n, fd.mul) >> fd.shift;
    return fd.mul == 0 ? n : q;
}

// ---------------------------------------------------------------------------
// Wavefront reductions with DPP (no LDS traffic for the first four steps).
// ---------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(
        __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <-> 7-i inside each 8
constexpr int kDppRowMirror = 0x140;  // lane i <-> 15-i inside each 16

// Sum over aligned teams of TL lanes (TL = 4, 8, 16, 32 or 64); every lane of a
// team ends with the team total, added in the same order in every lane pair.
template <int TL>
__device__ __forceinline__ float team_sum(float v) {
    static_assert(TL == 4 || TL == 8 || TL == 16 || TL == 32 || TL == 64, "team size");
    v += dpp_move<kDppXor1>(v);
    v += dpp_move<kDppXor2>(v);
    if (TL >= 8) v += dpp_move<kDppHalfMirror>(v);
    if (TL >= 16) v += dpp_move<kDppRowMirror>(v);
    if (TL >= 32)  // swap 16-lane rows inside each 32: ds_swizzle bit mode, xor 0x10
        v += __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F));
    if (TL >= 64) {
        const float lo = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
        const float hi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
        v = lo + hi;
    }
    return v;
}

__device__ __forceinline__ float wave_sum(float v) { return team_sum<64>(v); }

// Maximum over aligned teams of TL lanes, same exchange pattern as team_sum.
template <int TL>
__device__ __forceinline__ float team_max(float v) {
    static_assert(TL == 4 || TL == 8 || TL == 16 || TL == 32 || TL == 64, "team size");
    v = fmaxf(v, dpp_move<kDppXor1>(v));
    v = fmaxf(v, dpp_move<kDppXor2>(v));
    if (TL >= 8) v = fmaxf(v, dpp_move<kDppHalfMirror>(v));
    if (TL >= 16) v = fmaxf(v, dpp_move<kDppRowMirror>(v));
    if (TL >= 32) v = fmaxf(v, __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F)));
    if (TL >= 64) {
        const float lo = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
        const float hi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
        v = fmaxf(lo, hi);
    }
    return v;
}

// Sum over a workgroup of NW wavefronts; `slots` is NW floats of LDS that no
// other reduction in flight uses.  One barrier; every thread gets the total.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float *slots) {
    const float w = wave_sum(v);
    if (NW == 1) return w;
    const int tid = threadIdx.x;
    if ((tid & (kWave - 1)) == 0) slots[tid / kWave] = w;
    __syncthreads();
    float t = 0.0f;
#pragma unroll
    for (int i = 0; i < NW; i++) t += slots[i];
    return t;
}

// ---------------------------------------------------------------------------
// Activation math (float32).
// ---------------------------------------------------------------------------
constexpr float kLog2e = 1.44269504088896340736f;

// x * 1/(1+exp(-x)); exp through the hardware 2^x, reciprocal through v_rcp_f32
// (both about 1 ulp): relative error of the result stays below 1e-6.
__device__ __forceinline__ float silu_f(float x) {
    const float e = __builtin_amdgcn_exp2f(-kLog2e * x);
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}

__device__ __forceinline__ float quick_gelu_f(float x) {
    const float e = __builtin_amdgcn_exp2f((-kLog2e * 1.702f) * x);
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// gelu(x) = x * Phi(x) = max(x, 0) - h(|x|) with h(t) = 0.5 * t * erfc(t / sqrt 2), written
// as 0.5 * (x + |x|) - t * 2^(t * P(t) - 1): neither tail cancels, one v_exp_f32, no branch.
// P is the degree-7 fit of log2(erfc(t / sqrt 2)) / t that minimises the absolute error of h
// (fit_gelu_poly.py next to this file prints these constants); its leading coefficient is
// negative, so the power of two vanishes beyond the fitted range by itself.  t is clamped to
// 64 (h is zero to float32 from 14 on) so that an infinite input gives gelu(inf) = inf and not
// inf * 0; NaN comes through the x + |x| term.  Against float64 the result is within 2.5e-7
// absolute everywhere (the float32 expression x * 0.5 * (1 + erff(x * sqrt 0.5)): 4.5e-7).
__device__ __forceinline__ float gelu_erf_f(float x) {
    const float t = fminf(fabsf(x), 64.0f);
    float p = -1.902064014e-06f;
    p = fmaf(p, t, 2.805691838e-05f);
    p = fmaf(p, t, -1.314731053e-04f);
    p = fmaf(p, t, -2.720760531e-04f);
    p = fmaf(p, t, 7.245421875e-03f);
    p = fmaf(p, t, -5.262761191e-02f);
    p = fmaf(p, t, -4.591621459e-01f);
    p = fmaf(p, t, -1.151111007e+00f);
    const float half_erfc = __builtin_amdgcn_exp2f(fmaf(p, t, -1.0f));
    return fmaf(x + fabsf(x), 0.5f, -(t * half_erfc));
}

struct OpCopy {
    static __device__ __forceinline__ float apply(float x) { return x; }
};
struct OpSilu {
    static __device__ __forceinline__ float apply(float x) { return silu_f(x); }
};
struct OpGelu {
    static __device__ __forceinline__ float apply(float x) { return gelu_erf_f(x); }
};
struct OpQuickGelu {
    static __device__ __forceinline__ float apply(float x) { return quick_gelu_f(x); }
};

}  // namespace msd
