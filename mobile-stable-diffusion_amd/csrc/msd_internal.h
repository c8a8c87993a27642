// Host-side declarations shared by the translation units of libmsd_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <atomic>
#include <stddef.h>
#include <stdint.h>
#include <tuple>
#include <utility>

#include "../../include/msd_hip.h"

namespace msd {

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Kernel launches go through hipLaunchKernel, which returns the status of that launch itself;
// nothing reads or clears the thread's "last error" of the HIP runtime, so an error that an
// unrelated earlier call of the application left there is neither reported as ours nor lost.
// launch() keeps the first failure of the calling thread's launches until launch_status()
// returns it (and forgets it): a dispatcher launches, then returns launch_status().
inline thread_local hipError_t t_launch_error = hipSuccess;

template <typename... KArgs, typename... Args, size_t... I>
inline hipError_t launch_with(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds, hipStream_t stream,
                              std::index_sequence<I...>, Args &&...args) {
    std::tuple<KArgs...> values(static_cast<KArgs>(std::forward<Args>(args))...);
    void *pointers[sizeof...(KArgs) + 1] = {const_cast<void *>(static_cast<const void *>(&std::get<I>(values)))..., nullptr};
    return hipLaunchKernel(reinterpret_cast<const void *>(kernel), grid, block, pointers, lds, stream);
}

template <typename... KArgs, typename... Args>
inline void launch(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds, hipStream_t stream, Args &&...args) {
    static_assert(sizeof...(KArgs) == sizeof...(Args), "one argument per kernel parameter");
    const hipError_t err = launch_with(kernel, grid, block, lds, stream, std::index_sequence_for<KArgs...>{},
                                       std::forward<Args>(args)...);
    if (err != hipSuccess && t_launch_error == hipSuccess) t_launch_error = err;
}

inline int launch_status() {
    const hipError_t err = t_launch_error;
    t_launch_error = hipSuccess;
    return (int)err;
}

// ---- GroupNorm scratch: what workgroups sharing one (sample, group) exchange ----
constexpr uint32_t kGnMaxSplit = 64;    // workgroups per unit (one wavefront reads all slots)
constexpr uint32_t kGnMaxUnits = 8192;  // units that own scratch slots; larger launches never split

// ---- what the GroupNorm register kernels are built for (kernels: groupnorm.hip, plan: gn_plan.hip) ----
constexpr int kGnMaxThreads = 1024;
constexpr int kGnMaxK = 20;             // vectors per lane; the largest only for slices it fits exactly
constexpr int kGnMaxRaggedK = 16;       // the largest with code for a ragged slice
constexpr int kGnSharedMaxK = 10;       // kernels with several writers per unit exist up to this many vectors per lane
constexpr int kGnPrefetchAffineK = 6;   // vectors per lane up to which gamma / beta are kept in registers
constexpr uint32_t kGnLdsChannels = 1024;  // channels per group the LDS copy of gamma / beta has room for

struct GnScratch {
    unsigned long long *slot_mean;  // [kGnMaxUnits][kGnMaxSplit]  (tag << 32) | float bits
    unsigned long long *slot_m2;    // [kGnMaxUnits][kGnMaxSplit]
    uint32_t *epoch;                // [kGnMaxUnits] launches completed on this unit
    uint32_t *done;                 // [kGnMaxUnits] slices finished in the running launch
    uint32_t *fallbacks;            // [1] slices that stopped waiting and computed a sibling's statistics themselves
    uint32_t units;                 // units the arrays above have room for
};

// Per-(device, stream) scratch, created on first use (hipMalloc + hipMemset).
hipError_t get_scratch(hipStream_t stream, GnScratch *out);
// The fixed scratch inside the code object (no allocation), shared by all streams of a device.
hipError_t get_static_scratch(GnScratch *out);

// Tuning overrides set through msd_set_tuning (0 = choose automatically).  Atomics: a launch
// on one thread may read them while another thread sets them; each launch reads a knob once.
struct Tuning {
    std::atomic<int> gn_split{0};
    std::atomic<int> gn_threads{0};
    std::atomic<int> gn_writers{0};
    std::atomic<int> ln_chunk{0};
    std::atomic<int> ln_threads{0};
    std::atomic<int> geglu_vectors{0};
    std::atomic<int> act_vectors{0};
    std::atomic<int> softmax_rows{0};
    std::atomic<int> gn_spin_limit{0};
    std::atomic<int> device_cus{0};
    std::atomic<int> device_xcds{0};
    std::atomic<int> gn_plan_rule_only{0};
};
extern Tuning g_tuning;

// The launch msd_groupnorm makes for a shape (see gn_decide in gn_plan.hip): split == 0 is the
// general kernel, otherwise split workgroups of `threads` lanes per (sample, group), k 16-byte
// vectors per lane, vec_per_slice vectors per workgroup.
struct GnDecision {
    uint32_t split;
    uint32_t threads;
    uint32_t k;
    uint32_t vec_per_slice;
    uint32_t writers;  // workgroups per whole unit that each store a part of it (1: the usual launch)
};
GnDecision gn_decide(size_t elt, size_t batch, size_t channels, size_t hw, size_t groups, bool aligned,
                     size_t max_units, bool may_share);

// Compute units and XCDs of the current device (gn_plan.hip; the knobs can replace them).
struct Chip {
    uint32_t cus;
    uint32_t xcds;
};
Chip chip_info();
// Lanes and vectors per lane (k == 0: none fits) for a workgroup that holds `vecs` vectors.
struct GnThreads {
    uint32_t threads;
    int k;
};
int gn_k_for(uint32_t vecs, uint32_t threads, uint32_t max_k, bool equal_slices);
GnThreads gn_threads_for(const Chip &chip, size_t elt, uint32_t vecs, uint32_t split, size_t blocks, uint32_t max_k,
                         bool equal_slices, bool shared);
uint32_t gn_auto_writers(const Chip &chip, size_t elt, size_t units, size_t vec_per_unit);

// ---- per-dtype dispatchers (T = float or __half), defined in the kernel files ----
// fixed: scratch to use instead of the stream's own (units beyond its capacity are refused)
template <typename T>
int gn_dispatch(const void *x, const void *chunk, void *y, const float *gamma, const float *beta,
                size_t batch, size_t channels, size_t hw, size_t groups, float eps, bool silu,
                const GnScratch *fixed, hipStream_t stream);
// y is token-major [batch, hw, channels]; must not overlap x
template <typename T>
int gn_tokens_dispatch(const void *x, void *y, const float *gamma, const float *beta, size_t batch,
                       size_t channels, size_t hw, size_t groups, float eps, hipStream_t stream);
// res / sum may be null (plain LayerNorm); otherwise sum = x + res is written and normalised
template <typename T>
int ln_dispatch(const void *x, const void *res, void *sum, void *y, const float *gamma,
                const float *beta, size_t rows, size_t dim, float eps, hipStream_t stream);
template <typename T>
int add_dispatch(const void *a, const void *b, void *c, size_t n, size_t chunk_size,
                 hipStream_t stream);  // chunk_size 0: elementwise; else b holds one value per chunk
template <typename T>
int geglu_dispatch(const void *proj, void *out, size_t rows, size_t inner, hipStream_t stream);

template <typename T>
int permute_021_dispatch(const void *src, void *dst, size_t isize, size_t jsize, size_t ksize,
                         hipStream_t stream);

enum class Act { Silu, Gelu, QuickGelu, Copy };
template <typename T>
int act_dispatch(Act op, const void *x, void *y, size_t n, hipStream_t stream);
template <typename T>
int temb_dispatch(const int64_t *timesteps, void *out, size_t batch, size_t dim, float max_period,
                  hipStream_t stream);

// y[m, n] = act_out(act_in(x) . w^T + bias), m <= 8; activations: 0 none, 1 SiLU
template <typename T>
int linear_rows_dispatch(const void *x, const void *w, const float *bias, void *y, size_t m, size_t n,
                         size_t k, int act_in, int act_out, hipStream_t stream);
// `count` Linear layers on the same rows x; ws / biases / ys / ns are host arrays
template <typename T>
int linear_rows_grouped_dispatch(const void *x, const void *const *ws, const float *const *biases,
                                 void *const *ys, const size_t *ns, size_t count, size_t m, size_t k,
                                 int act_in, int act_out, hipStream_t stream);
template <typename T>
int softmax_dispatch(const void *x, void *y, size_t rows, size_t cols, int stable, hipStream_t stream);
template <typename T>
int ddim_update_dispatch(const void *x, const void *e_t, void *x_prev, size_t n, float a_t,
                         float a_prev, float sqrt_one_minus_at, hipStream_t stream);

}  // namespace msd
