/*
 * CPU oracle for the norm / activation / embedding path.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP kernels are
 * compared against and the "port" CPU baseline a benchmark may time.  Nothing
 * in the shipped product path may link, load or call it.
 *
 * Every orc_* function restates, in float32 and in the same operation order,
 * one OpenCL kernel or host loop of the reference (paths are relative to
 * /root/reference/app/src/main; K/ = assets/kernel/, M/ = cpp/modules/).  The
 * orc64_* functions are independent float64 textbook versions of the same
 * mathematics, used to pin the restatements.
 *
 * Pinning status (what checks each function, all in tests/test_oracle_*.py):
 *   orc_group_*, orc_groupnorm_forward : torch.nn.functional.group_norm fixtures,
 *        orc64 brute force, constant-input and unit-variance invariants.
 *   orc_layer_*, orc_layernorm_forward : torch.nn.functional.layer_norm fixtures,
 *        orc64 brute force, invariants.
 *   orc_silu, orc_gelu, orc_gelu_multiply : torch fixtures, closed-form known
 *        values, gelu(x)-gelu(-x)=x, half-order test for gelu_multiply.
 *   orc_timestep_embedding : t=0 and i=0 closed forms, cos^2+sin^2=1, float64
 *        cross-check, torch float32 fixture of the textbook formula.
 *   orc_ddim_timesteps : closed form 1+c*k and the reference's shipped
 *        literal 981 (native-lib.cpp:240) as the first step of 50.
 *   orc_elemwise_add, orc_chunkwise_add, orc_permute3D_0_2_1 : exact; checked against numpy
 *        broadcasting / transpose (bit-exact).
 *   orc_linear : torch.nn.functional.linear fixtures (non-square, with and without
 *        bias), orc64 brute force, one-hot rows that select single weights.
 *   orc_softmax : torch.softmax fixtures, rows sum to 1, shift invariance against the
 *        max-subtracting float64 textbook form, odd workgroup sizes against a plain sum.
 *   orc_alphas_cumprod, orc_ddim_schedule : the LDM "linear" beta schedule computed by
 *        torch in float64 (fixture), first / last known values, alphas_prev shift.
 *   orc_ddim_update : float64 fixture of the LDM DDIM step (eta 0), e_t = 0 and
 *        a_prev = a_t special cases.
 *   orc_quick_gelu : PARITY UNPINNED BY THE REFERENCE (the reference has no
 *        quick_GELU); pinned only by the closed form x*sigmoid(1.702x).
 */
#ifndef MSD_ORACLE_H
#define MSD_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- seeded synthetic data (own generator: splitmix64 + Box-Muller) ---- */
void orc_fill_normal(float *out, size_t n, uint64_t seed, float mean, float sigma);
/* replace ~1% of the elements by +/-20 (sign from the hash) */
void orc_add_outliers(float *x, size_t n, uint64_t seed, float magnitude);
void orc_fill_uniform_int(int64_t *out, size_t n, uint64_t seed, int64_t lo, int64_t hi_inclusive);

/* ---- IEEE binary16 storage emulation (round-to-nearest-even) ---- */
uint16_t orc_float_to_half_bits(float f);
float orc_half_bits_to_float(uint16_t h);
void orc_round_to_half(float *x, size_t n);                 /* x = float(half(x)) in place */
void orc_to_half_bits(const float *x, uint16_t *h, size_t n);
void orc_from_half_bits(const uint16_t *h, float *x, size_t n);

/* ---- faithful float32 restatements ---- */
/* K/group_norm.cl:1-27 and K/layer_norm.cl:1-27: one 64-lane workgroup per unit */
void orc_local_reduction_mean(const float *input, float *output, size_t n_workgroups,
                              size_t reduction_size);
/* K/group_norm.cl:29-57 and K/layer_norm.cl:29-56 */
void orc_local_reduction_variance(const float *input, const float *mean, float *output,
                                  size_t n_workgroups, size_t reduction_size);
/* K/group_norm.cl:59-76 */
void orc_group_norm(const float *input, const float *mean, const float *variance,
                    const float *weight, const float *bias, size_t group_size,
                    size_t channel_size, float epsilon, float *output, size_t n);
/* K/layer_norm.cl:58-78 (epsilon is a __constant 1e-5 there; a parameter here) */
void orc_layer_norm(const float *input, const float *mean, const float *variance,
                    const float *weight, const float *bias, size_t chunk_size,
                    float epsilon, float *output, size_t n);
/* K/util.cl:124-134 */
void orc_silu(const float *src, float *dst, size_t n);
/* K/util.cl:104-122 */
void orc_gelu(const float *src, float *dst, size_t n);
/* closed form x*sigmoid(1.702x); not in the reference */
void orc_quick_gelu(const float *src, float *dst, size_t n);
/* K/util.cl:1-12 */
void orc_elemwise_add(const float *a, const float *b, float *c, size_t n);
/* K/util.cl:136-148: c[i] = a[i] + chunk[i / chunk_size] */
void orc_chunkwise_add(const float *a, const float *chunk, float *c, size_t n, size_t chunk_size);
/* K/util.cl:47-64: [i, j, k] -> [i, k, j] */
void orc_permute3D_0_2_1(const float *src, float *dst, size_t isize, size_t jsize, size_t ksize);
/* K/geglu.cl:1-25: value = first half of a row, gate = second half */
void orc_gelu_multiply(const float *ab, float *dst, size_t rows, size_t inner);
/* M/UNetModel.cpp:1935-1958 */
void orc_timestep_embedding(int64_t timestep, float *out, int dim, float max_period);
/* frequencies alone (the float32 expression at M/UNetModel.cpp:1950) */
void orc_timestep_freqs(float *freq, int half, float max_period);
/* M/DDIMSampler.cpp:60-64 (ascending list) ; returns the count, writes at most cap */
int orc_ddim_timesteps(int ddim_num_steps, int *out, int cap);

/* ---- host-object drivers: the call sequence of the reference's forward() ---- */
/* M/nn/GroupNorm.cpp:75-145 applied per sample (the reference is batch 1), then
 * optionally the separate silu pass of M/nn/ResBlock.cpp:136-142.  Returns 0, or
 * -1 when a reference precondition (M/nn/GroupNorm.cpp:83-93) is violated. */
int orc_groupnorm_forward(const float *x, float *y, const float *weight, const float *bias,
                          size_t batch, size_t channels, size_t hw, size_t groups, float eps,
                          int silu);
/* M/nn/LayerNorm.cpp:73-139 ; -1 when dim % 64 != 0 (M/nn/LayerNorm.cpp:61) */
int orc_layernorm_forward(const float *x, float *y, const float *weight, const float *bias,
                          size_t rows, size_t dim, float eps);

/* ---- float64 textbook versions (independent of the restatements) ---- */
void orc64_groupnorm(const float *x, double *y, const float *weight, const float *bias,
                     size_t batch, size_t channels, size_t hw, size_t groups, double eps,
                     int silu);
void orc64_layernorm(const float *x, double *y, const float *weight, const float *bias,
                     size_t rows, size_t dim, double eps);
void orc64_silu(const float *x, double *y, size_t n);
void orc64_gelu(const float *x, double *y, size_t n);
void orc64_quick_gelu(const float *x, double *y, size_t n);
void orc64_geglu(const float *ab, double *y, size_t rows, size_t inner);
void orc64_timestep_embedding(int64_t timestep, double *out, int dim, double max_period);

/* ---- neighbours of the path (the callers either side of it) ---- */
/* K/linear.cl:345-430 via M/nn/Linear.cpp:244-289: c[m,n] = a[m,k] . w[n,k]^T + bias; bias may be NULL */
void orc_linear(const float *a, const float *w, const float *bias, float *c, size_t m, size_t n,
                size_t k);
void orc64_linear(const float *a, const float *w, const float *bias, double *c, size_t m, size_t n,
                  size_t k);
/* K/util.cl:150-187 with a workgroup of local_size (<= 1024) lanes per chunk */
void orc_softmax(const float *input, float *output, size_t rows, size_t chunk_size,
                 size_t local_size);
void orc64_softmax(const float *input, double *output, size_t rows, size_t chunk_size);
/* M/DDIMSampler.cpp:18-39: out[1000] */
void orc_alphas_cumprod(float *out);
/* M/DDIMSampler.cpp:60-76,123-137; returns the count (-1 bad steps, -2 table overrun) */
int orc_ddim_schedule(int ddim_num_steps, int *timesteps, float *alphas, float *alphas_prev,
                      float *sqrt_one_minus_alphas, int cap);
/* M/DDIMSampler.cpp:94-121 */
void orc_ddim_update(const float *x, const float *e_t, float *x_prev, size_t n, float a_t,
                     float a_prev, float sqrt_one_minus_at);
void orc64_ddim_update(const float *x, const float *e_t, double *x_prev, size_t n, double a_t,
                       double a_prev);

/* ---- threading control for the CPU-baseline leg ---- */
int orc_max_threads(void);
void orc_set_threads(int n);

#ifdef __cplusplus
}
#endif
#endif
