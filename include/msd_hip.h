/*
 * msd_hip.h - C ABI of the MI355X (gfx950) norm / activation / embedding kernels.
 *
 * Plain C: pointers, sizes, ints.  Every device pointer is HIP device memory on
 * the current device; `stream` is a hipStream_t passed as void* (NULL = the
 * default stream).  Calls are asynchronous on that stream.  Return value: 0 on
 * success, otherwise a hipError_t value (1 = hipErrorInvalidValue is also used
 * for rejected shapes / null pointers / unknown dtype).  No call throws.
 * Where an output may take the place of an input ("may alias") it must be exactly
 * that input or lie apart from it, and where it must not overlap an input no byte
 * may be shared: any other overlap is refused with hipErrorInvalidValue before
 * anything is launched.
 *
 * Each entry point names the reference interface it replaces (paths relative to
 * app/src/main of 9Hyeonwoo/mobile-stable-diffusion; K/ = assets/kernel/,
 * M/ = cpp/modules/).  The reference is fp32, batch 1; `dtype` and `batch` are
 * extensions.  gamma / beta are always float32.
 */
#ifndef MSD_HIP_H
#define MSD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MSD_OK 0
#define MSD_ERR_INVALID_VALUE 1 /* == hipErrorInvalidValue */
#define MSD_ERR_SCRATCH_LIMIT (-2) /* msd_groupnorm_noalloc: batch * groups above its fixed scratch */

/* storage type of activations; arithmetic is always float32 */
#define MSD_DTYPE_F32 0
#define MSD_DTYPE_F16 1

/* Library version: major*10000 + minor*100 + patch. */
int msd_version(void);

/* Human-readable text for a return code (static storage). */
const char *msd_error_string(int code);

/*
 * Creates the per-(device, stream) scratch (a few MiB, holds the partial
 * statistics that workgroups sharing one GroupNorm group exchange) ahead of
 * time.  Optional: msd_groupnorm creates it on first use; call this first
 * when the first msd_groupnorm on a stream would otherwise happen under
 * stream capture.  A graph captured on a stream keeps using that stream's
 * scratch: GroupNorm launches that share scratch must not run concurrently
 * (do not replay such a graph on a second stream while the first is busy with
 * GroupNorms).  Also looks up the device address of msd_groupnorm_noalloc's fixed
 * scratch on the current device.  hipStreamPerThread is refused (one handle, a
 * different stream in every thread) - here and by msd_groupnorm, msd_chunk_add_groupnorm
 * and msd_groupnorm_tokens for every shape, whether or not that launch would need the
 * scratch; msd_groupnorm_noalloc, which has its own, takes it.  No reference counterpart
 * (the reference allocates two temporaries per forward, M/nn/GroupNorm.cpp:95-103).
 */
int msd_init(void *stream);

/* Frees the scratch of `stream` on the current device (for applications that create and
 * destroy streams; the stream must be idle).  The next GroupNorm on it creates it again. */
int msd_release(void *stream);

/* Frees every scratch buffer created so far on all devices.  Call it only when no
 * msd_groupnorm* launch is still in flight (synchronise the streams first); the next
 * GroupNorm creates its scratch again. */
int msd_shutdown(void);

/*
 * Synchronises `stream`; returns 0 or the HIP error the stream reports.  No reference
 * counterpart (the reference blocks in clFinish, M/UNetModel.cpp:1830).
 */
int msd_status(void *stream);

/*
 * Diagnostic.  Workgroups that share one (sample, group) exchange partial statistics; one
 * that does not receive a sibling's within its poll limit computes them itself from the
 * input, so the output is right either way.  This synchronises `stream` and returns in
 * *count how often that happened so far on the stream's scratch and on the fixed scratch of
 * msd_groupnorm_noalloc (0 on an idle GPU); reset != 0 clears the counters.
 */
int msd_gn_fallbacks(void *stream, unsigned int *count, int reset);

/*
 * Tuning / test knobs (process-wide; value 0 restores the automatic choice).  They change
 * how a launch is cut into workgroups, never its result.  Each launch reads a knob once
 * (atomically), so setting one while another thread launches is safe but affects that
 * thread's later launches.  No reference counterpart.
 */
#define MSD_TUNE_GN_SPLIT 0      /* workgroups per (sample, group): power of two <= 64 */
#define MSD_TUNE_GN_THREADS 1    /* GroupNorm workgroup size: multiple of 64, <= 1024 */
#define MSD_TUNE_LN_CHUNK 2      /* bytes a LayerNorm lane moves per load: 8 or 16 */
#define MSD_TUNE_LN_THREADS 3    /* LayerNorm workgroup size: 64, 128, 256 or 512 */
#define MSD_TUNE_GEGLU_VECTORS 4 /* 16-byte vectors per GEGLU lane: 1, 2 or 4 */
#define MSD_TUNE_ACT_VECTORS 5   /* 16-byte vectors per lane of SiLU / GELU / quick_GELU: 1, 2 or 4 */
#define MSD_TUNE_SOFTMAX_ROWS 6   /* rows per workgroup of the short-row softmax: 16, 32 or 64 */
#define MSD_TUNE_GN_SPIN_LIMIT 7  /* polls a GroupNorm workgroup waits for a sibling before it computes
                                     that sibling's statistics itself (tests set 1 to exercise that path) */
#define MSD_TUNE_GN_WRITERS 8     /* workgroups that share one whole (sample, group), each storing a part
                                     of it: 1 (never), 2, 4, 8 or 16 (wherever the launch allows it) */
#define MSD_TUNE_DEVICE_CUS 9     /* plan GroupNorm launches for a chip of this many compute units instead of
                                     asking the current device (tests; 0: ask) */
#define MSD_TUNE_DEVICE_XCDS 10   /* ... and of this many XCDs, each with an L2 of its own (0: ask) */
#define MSD_TUNE_GN_PLAN_RULE_ONLY 11 /* 1: ignore the table of measured GroupNorm plans, plan by the rule alone
                                     (benchmark sweeps measure the rule with it) */
int msd_set_tuning(int knob, int value);

/*
 * GroupNorm over NCHW, optionally followed by SiLU, in one launch.
 * Replaces the 3-kernel chain enqueued by GroupNorm::forward
 * (M/nn/GroupNorm.cpp:105-145; K/group_norm.cl:1-76) and, with fuse_silu != 0,
 * the separate silu enqueue that follows it (M/nn/ResBlock.cpp:136-142,
 * K/util.cl:124-134).  Biased variance, y = fma((x-mean)/sqrt(var+eps), gamma[c],
 * beta[c]).  x and y are [batch, channels, hw]; y may alias x exactly (in place,
 * M/nn/ResBlock.cpp:222).  Requires channels % groups == 0.  When y lies apart from x
 * and there are fewer than 256 (sample, group) units, several workgroups share each unit
 * (msd_groupnorm_plan tells); the statistics are then summed in another order than for the
 * call in place, so the two results can differ in the last bit.  A given call is
 * reproducible bit for bit as long as msd_gn_fallbacks() stays 0: a workgroup that stopped
 * waiting for a sibling sums that sibling's part in another order (same accuracy).
 */
int msd_groupnorm(const void *x, void *y, const float *gamma, const float *beta,
                  size_t batch, size_t channels, size_t hw, size_t groups, float eps,
                  int fuse_silu, int dtype, void *stream);

/*
 * msd_groupnorm for callers that cannot allocate (code under stream capture, tight serving
 * loops, harnesses that forbid hipMalloc): same arguments, same kernels, same result bit for
 * bit (while msd_gn_fallbacks() stays 0, see msd_groupnorm), but the workgroups' exchange
 * area is a fixed 1 MiB array inside the library's code
 * object instead of a per-stream allocation, so the call never allocates or frees (its first
 * call on a device looks the array's address up; msd_init does that ahead of time).  Limit:
 * batch * groups <= 1024, otherwise MSD_ERR_SCRATCH_LIMIT.  Every stream of a device shares
 * the one array: calls that overlap in time on one GPU race (their results are undefined);
 * calls ordered by a stream or by events are fine, and nothing needs clearing between them.
 * Each GPU holds its array until the process ends.  No counterpart in the reference.
 */
int msd_groupnorm_noalloc(const void *x, void *y, const float *gamma, const float *beta,
                          size_t batch, size_t channels, size_t hw, size_t groups, float eps,
                          int fuse_silu, int dtype, void *stream);

/*
 * The launch msd_groupnorm (noalloc != 0: msd_groupnorm_noalloc) makes for this shape on 16-byte
 * aligned tensors, under the tuning knobs as they are set: *split workgroups per (sample, group),
 * *threads lanes each, *vectors_per_lane 16-byte vectors held per lane.  *writers > 1 (then
 * *split = 1): that many workgroups per (sample, group) each load and reduce all of it and store
 * one part; such a launch is only made when y does not overlap x, so in_place != 0 asks for the
 * plan of a call with y == x.  *split = 0 (the others too) means the general kernel: one 256-lane
 * workgroup per (sample, group), nothing held in registers.  Host arithmetic only: needs no GPU
 * and launches nothing.  For diagnostics, tests and benchmark tables.  No counterpart in the
 * reference (its geometry is fixed, M/nn/GroupNorm.cpp:105-128).
 */
int msd_groupnorm_plan(size_t batch, size_t channels, size_t hw, size_t groups, int dtype, int noalloc,
                       int in_place, int *split, int *threads, int *vectors_per_lane, int *writers);

/*
 * GroupNorm whose result is stored token-major: x is [batch, channels, hw], y is
 * [batch, hw, channels], y[b, p, c] = GroupNorm(x)[b, c, p].  Replaces GroupNorm::forward
 * followed by the permute3D_0_2_1 enqueue of SpatialTransformer::forward
 * (M/nn/SpatialTransformer.cpp:127-139; K/util.cl:47-64) in one launch; equal to
 * msd_groupnorm + that permute up to the summation order of the statistics (a few float
 * ulps).  No SiLU (the reference has none there; its eps is 1e-6).  y must not overlap x.
 */
int msd_groupnorm_tokens(const void *x, void *y, const float *gamma, const float *beta, size_t batch,
                         size_t channels, size_t hw, size_t groups, float eps, int dtype,
                         void *stream);

/*
 * dst[i, k, j] = src[i, j, k]: the permute3D_0_2_1 kernel (K/util.cl:47-64) that
 * SpatialTransformer::forward enqueues between NCHW and token layout
 * (M/nn/SpatialTransformer.cpp:132-139,157-164).  dst must not overlap src.
 */
int msd_permute_0_2_1(const void *src, void *dst, size_t isize, size_t jsize, size_t ksize, int dtype,
                      void *stream);

/*
 * LayerNorm over the last dimension of a row-major [rows, dim] tensor.
 * Replaces LayerNorm::forward (M/nn/LayerNorm.cpp:94-139; K/layer_norm.cl:1-78);
 * the reference's eps is the constant 1e-5 (K/layer_norm.cl:58).  y may alias x.
 */
int msd_layernorm(const void *x, void *y, const float *gamma, const float *beta, size_t rows,
                  size_t dim, float eps, int dtype, void *stream);

/*
 * The two additions the reference runs right before its norms, and their fusions.
 *   msd_elemwise_add   c[i] = a[i] + b[i]                 K/util.cl:1-12 (the residual adds
 *                      of M/nn/BasicTransformerBlock.cpp:126-134,149-156,170-177)
 *   msd_chunkwise_add  c[i] = a[i] + chunk[i / chunk_size] K/util.cl:136-148 (the time-embedding
 *                      add of M/nn/ResBlock.cpp:188-199; chunk holds one value per run of
 *                      chunk_size elements, i.e. [batch, channels] with chunk_size = hw)
 * c may alias a (every reference call site does) or b.
 *
 *   msd_chunk_add_groupnorm  = msd_chunkwise_add(x, chunk, tmp, ., hw) followed by
 *                      msd_groupnorm(tmp, y, ...), bit for bit (while msd_gn_fallbacks() stays
 *                      0, see msd_groupnorm), without the pass over tmp: replaces
 *                      M/nn/ResBlock.cpp:188-199 + 222-232 in one launch.  chunk is
 *                      [batch, channels] in the activation storage type and must not overlap y.
 *   msd_add_layernorm  = msd_elemwise_add(a, b, sum) followed by msd_layernorm(sum, y, ...), bit
 *                      for bit, in one launch; `sum` is written because the reference keeps it
 *                      as the next residual (M/nn/BasicTransformerBlock.cpp:126-136,149-158).
 *                      sum may alias a or b.
 */
int msd_elemwise_add(const void *a, const void *b, void *c, size_t n, int dtype, void *stream);
int msd_chunkwise_add(const void *a, const void *chunk, void *c, size_t n, size_t chunk_size,
                      int dtype, void *stream);
int msd_chunk_add_groupnorm(const void *x, const void *chunk, void *y, const float *gamma,
                            const float *beta, size_t batch, size_t channels, size_t hw,
                            size_t groups, float eps, int fuse_silu, int dtype, void *stream);
int msd_add_layernorm(const void *a, const void *b, void *sum, void *y, const float *gamma,
                      const float *beta, size_t rows, size_t dim, float eps, int dtype,
                      void *stream);

/*
 * GEGLU epilogue on an already projected tensor: proj is [rows, 2*inner] with
 * the value in the first half of each row and the gate in the second;
 * out[r, c] = proj[r, c] * gelu_erf(proj[r, inner + c]).  Replaces the
 * gelu_multiply enqueue of GEGLU::forward (M/nn/GEGLU.cpp:71-78; K/geglu.cl:1-25).
 * out must not overlap proj.
 */
int msd_geglu(const void *proj, void *out, size_t rows, size_t inner, int dtype, void *stream);

/*
 * Elementwise activations over n elements; y may alias x (every reference call
 * site is in place).
 *   msd_silu       K/util.cl:124-134 (enqueued at M/nn/ResBlock.cpp:136-142,173-180,
 *                  225-232; M/UNetModel.cpp:1110-1117,1803-1810)
 *   msd_gelu       K/util.cl:104-122 (M/nn/ResidualAttentionBlock.cpp:146-153), erf form
 *   msd_quick_gelu x*sigmoid(1.702x); no reference counterpart
 */
int msd_silu(const void *x, void *y, size_t n, int dtype, void *stream);
int msd_gelu(const void *x, void *y, size_t n, int dtype, void *stream);
int msd_quick_gelu(const void *x, void *y, size_t n, int dtype, void *stream);

/*
 * Plain device copy of `bytes` (multiple of 4) with the same 16-byte streaming kernel the
 * activations use and no arithmetic.  Measurement helper with no reference counterpart: it
 * gives the bandwidth a read-once / write-once launch of a given size can reach on the
 * machine, the ceiling the other kernels are compared with, and calibrates traffic counters.
 */
int msd_copy(const void *src, void *dst, size_t bytes, void *stream);

/*
 * Sinusoidal timestep embedding, out[b] = [cos(t_b*f_i) | sin(t_b*f_i)],
 * f_i = exp(-log(max_period) * i / (dim/2)), i < dim/2.  Replaces the host loop
 * UNetModel::createTimestepEmbedding (M/UNetModel.cpp:1935-1958): same float32
 * expression for f_i and t*f_i.  timesteps is a device array of `batch` int64
 * values, out is [batch, dim]; dim must be even.
 */
int msd_timestep_embedding(const int64_t *timesteps, void *out, size_t batch, size_t dim,
                           float max_period, int dtype, void *stream);

/*
 * Integer DDIM timestep list (host only, no GPU work): c = 1000 / steps;
 * {1, 1+c, 1+2c, ...} while < 1000+1, ascending, exactly as
 * DDIMSampler::sample builds it (M/DDIMSampler.cpp:60-64); the sampler walks it
 * from the back (M/DDIMSampler.cpp:78-82).  Writes at most cap entries and
 * returns the full count, or -1 for steps outside [1, 1000].
 */
int msd_ddim_timesteps(int ddim_num_steps, int *out, int cap);

/*
 * Linear layer on the few rows of the time embedding: y[m, n] = act_out(act_in(x)[m, k] .
 * weight[n, k]^T + bias[n]), m <= 8 (larger m is a GEMM and is rejected).  x, weight and y
 * are in the storage type `dtype`, bias is float32 or NULL, accumulation is float32.
 * Replaces Linear::forward (M/nn/Linear.cpp:74-289, kernel K/linear.cl:345-430) at its
 * embedding call sites together with the silu enqueue next to it:
 *   act_out = MSD_ACT_SILU : time_embed_0 then silu   (M/UNetModel.cpp:1107-1117)
 *   no activation          : time_embed_2              (M/UNetModel.cpp:1119-1120)
 *   act_in = MSD_ACT_SILU  : silu(emb) then embed_linear, per ResBlock
 *                            (M/nn/ResBlock.cpp:173-183)
 * The reference adds the k products in ascending order into one accumulator; here each of
 * 64 lanes adds its share in ascending order and a fixed tree adds the lanes (agreement
 * within float32 summation error, see the tests).  y must not overlap x
 * (M/nn/Linear.cpp:78-81).
 */
#define MSD_ACT_NONE 0
#define MSD_ACT_SILU 1
int msd_linear_rows(const void *x, const void *weight, const float *bias, void *y, size_t m,
                    size_t n, size_t k, int act_in, int act_out, int dtype, void *stream);

/*
 * `count` such layers on the SAME rows x in one launch: ys[i][m, ns[i]] = act_out(act_in(x) .
 * weights[i][ns[i], k]^T + biases[i]).  weights, biases, ys and ns are host arrays of `count`
 * entries (device pointers / sizes); biases or any biases[i] may be NULL.  Replaces the 22
 * `silu(emb)` + `embed_linear->forward` pairs of one UNet step (M/nn/ResBlock.cpp:173-183),
 * which all read the one embedding that UNetModel::forward computes before its first block
 * (M/UNetModel.cpp:1107-1120), by one launch ahead of the blocks; each ys[i] equals what its
 * own msd_linear_rows call gives, bit for bit.  No ys[i] may overlap x, another ys[j], or
 * any weights[j] / biases[j] (the problems run side by side); n and k are at most 2^28.
 */
int msd_linear_rows_grouped(const void *x, const void *const *weights, const float *const *biases,
                            void *const *ys, const size_t *ns, size_t count, size_t m, size_t k,
                            int act_in, int act_out, int dtype, void *stream);

/*
 * Row softmax over the last dimension of [rows, cols]; y may alias x (every reference
 * call site is in place).  Replaces the softmax kernel K/util.cl:150-187 enqueued by
 * CrossAttention::forward (M/nn/CrossAttention.cpp:362-377) and AttnBlock::forward
 * (M/nn/AttnBlock.cpp:196-206).  stable = 0 computes exp(x) / sum exp(x) as that kernel
 * does (overflowing to inf / nan where it does, x > 88.7); stable != 0 subtracts the row
 * maximum first, which is the same value wherever the former is finite.
 */
int msd_softmax(const void *x, void *y, size_t rows, size_t cols, int stable, int dtype,
                void *stream);

/*
 * DDIM sampler arithmetic (M/DDIMSampler.cpp).  Host only:
 *   msd_alphas_cumprod  the 1000 cumulative alpha products of the constructor (:18-39):
 *                       betas = linspace(sqrt(0.00085), sqrt(0.0120), 1000)^2 and the
 *                       running product of 1 - beta in double, stored as float.
 *   msd_ddim_schedule   msd_ddim_timesteps plus make_schedule (:123-137) and :68-71:
 *                       alphas[i] = cumprod[t_i], alphas_prev = {cumprod[0], cumprod[t_0],
 *                       ...}, sqrt_one_minus_alphas[i] = sqrt(1 - alphas[i]).  Writes at most
 *                       cap entries per array and returns the full count; -1 for steps
 *                       outside [1, 1000]; -2 when the list would contain 1000 (steps > 500),
 *                       where the reference indexes one past its table.
 * On the stream:
 *   msd_ddim_update     x_prev = sqrt(a_prev) * ((x - sqrt_one_minus_at * e_t) / sqrt(a_t))
 *                       + sqrt(1 - a_prev) * e_t, the three loops of p_sample_ddim (:107-118,
 *                       eta 0) in one pass, every operation rounded separately in that order
 *                       (bit-identical to the host loops for float32).  x_prev may alias x.
 *                       a_t must be > 0 and a_prev in [0, 1] (else invalid value).
 */
int msd_alphas_cumprod(float *out_1000);
int msd_ddim_schedule(int ddim_num_steps, int *timesteps, float *alphas, float *alphas_prev,
                      float *sqrt_one_minus_alphas, int cap);
int msd_ddim_update(const void *x, const void *e_t, void *x_prev, size_t n, float a_t,
                    float a_prev, float sqrt_one_minus_at, int dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MSD_HIP_H */
