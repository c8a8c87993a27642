/*
 * CPU oracle: float32 restatements of the reference's OpenCL kernels and host
 * loops for the norm / activation / embedding path, plus float64 textbook
 * versions.  TEST INFRASTRUCTURE ONLY - see oracle.h.
 *
 * Build: see oracle/Makefile (-ffp-contract=off so that a*b+c is never fused
 * unless the reference wrote fma()).  The outer "one workgroup" / "one work
 * item" loops carry OpenMP pragmas so the same code serves as the CPU
 * baseline; every unit is independent, so results do not depend on the
 * thread count.
 */
#include "oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define WORK_GROUP_SIZE 64 /* M/nn/GroupNorm.cpp:13, M/nn/LayerNorm.cpp:11 */

/* ------------------------------------------------------------------ */
/* synthetic data                                                      */
/* ------------------------------------------------------------------ */
static inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

static inline double u01(uint64_t h) { /* (0,1) */
    return ((double)(h >> 11) + 0.5) * (1.0 / 9007199254740992.0);
}

void orc_fill_normal(float *out, size_t n, uint64_t seed, float mean, float sigma) {
    const uint64_t base = splitmix64(seed);
    const size_t pairs = (n + 1) / 2;
#pragma omp parallel for schedule(static)
    for (size_t p = 0; p < pairs; p++) {
        const double u1 = u01(splitmix64(base + 2 * p));
        const double u2 = u01(splitmix64(base + 2 * p + 1));
        const double r = sqrt(-2.0 * log(u1));
        const double a = 6.283185307179586476925 * u2;
        out[2 * p] = (float)((double)mean + (double)sigma * r * cos(a));
        if (2 * p + 1 < n) out[2 * p + 1] = (float)((double)mean + (double)sigma * r * sin(a));
    }
}

void orc_add_outliers(float *x, size_t n, uint64_t seed, float magnitude) {
    const uint64_t base = splitmix64(seed ^ 0xA5A5A5A55A5A5A5Aull);
    for (size_t i = 0; i < n; i++) {
        const uint64_t h = splitmix64(base + i);
        if (h % 100 == 0) x[i] = ((h >> 40) & 1) ? magnitude : -magnitude;
    }
}

void orc_fill_uniform_int(int64_t *out, size_t n, uint64_t seed, int64_t lo,
                          int64_t hi_inclusive) {
    const uint64_t base = splitmix64(seed);
    const uint64_t span = (uint64_t)(hi_inclusive - lo) + 1;
    for (size_t i = 0; i < n; i++) out[i] = lo + (int64_t)(splitmix64(base + i) % span);
}

/* ------------------------------------------------------------------ */
/* binary16 emulation                                                  */
/* ------------------------------------------------------------------ */
uint16_t orc_float_to_half_bits(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | ((absx > 0x7F800000u) ? 0x0200u : 0));
    if (absx >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* rounds to inf */
    if (absx < 0x33000001u) return (uint16_t)sign;               /* rounds to zero */
    int exp = (int)(absx >> 23) - 127;
    uint32_t man = (absx & 0x007FFFFFu) | 0x00800000u; /* 24-bit significand */
    int shift;                                         /* bits dropped */
    uint32_t hexp;
    if (exp < -14) { /* subnormal half */
        shift = 13 + (-14 - exp);
        hexp = 0;
    } else {
        shift = 13;
        hexp = (uint32_t)(exp + 15);
    }
    uint32_t kept = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u);
    const uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (kept & 1u))) kept++;
    /* for normals kept carries the implicit bit at position 10 */
    uint32_t h = (hexp << 10) + kept - (hexp ? 0x400u : 0u);
    return (uint16_t)(sign | h);
}

float orc_half_bits_to_float(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1Fu;
    const uint32_t man = h & 0x3FFu;
    uint32_t x;
    if (exp == 0) {
        if (man == 0) {
            x = sign;
        } else { /* subnormal: value = man * 2^-24 */
            float v = (float)man * 5.9604644775390625e-8f;
            memcpy(&x, &v, 4);
            x |= sign;
        }
    } else if (exp == 31) {
        x = sign | 0x7F800000u | (man << 13);
    } else {
        x = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

void orc_round_to_half(float *x, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) x[i] = orc_half_bits_to_float(orc_float_to_half_bits(x[i]));
}

void orc_to_half_bits(const float *x, uint16_t *h, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) h[i] = orc_float_to_half_bits(x[i]);
}

void orc_from_half_bits(const uint16_t *h, float *x, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) x[i] = orc_half_bits_to_float(h[i]);
}

/* ------------------------------------------------------------------ */
/* faithful float32 restatements                                       */
/* ------------------------------------------------------------------ */

/* The 64-entry local-memory tree of K/group_norm.cl:17-22: offsets 32,16,..,1,
 * lane l adds lane l+offset. */
static inline float tree_reduce_64(float *sums) {
    for (int offset = WORK_GROUP_SIZE / 2; offset > 0; offset /= 2)
        for (int l = 0; l < offset; l++) sums[l] += sums[l + offset];
    return sums[0];
}

void orc_local_reduction_mean(const float *input, float *output, size_t n_workgroups,
                              size_t reduction_size) {
#pragma omp parallel for schedule(static)
    for (size_t wg = 0; wg < n_workgroups; wg++) {
        float sums[WORK_GROUP_SIZE];
        for (int l = 0; l < WORK_GROUP_SIZE; l++) {
            /* K/group_norm.cl:10-14: lane l walks i + j*localSize */
            const size_t i = wg * WORK_GROUP_SIZE * reduction_size + (size_t)l;
            float sum = 0.0f;
            for (size_t j = 0; j < reduction_size; j++) sum += input[i + j * WORK_GROUP_SIZE];
            sums[l] = sum;
        }
        /* K/group_norm.cl:24-26: divide by (localSize * reductionSize) as float */
        output[wg] = tree_reduce_64(sums) / (float)(WORK_GROUP_SIZE * reduction_size);
    }
}

void orc_local_reduction_variance(const float *input, const float *mean, float *output,
                                  size_t n_workgroups, size_t reduction_size) {
#pragma omp parallel for schedule(static)
    for (size_t wg = 0; wg < n_workgroups; wg++) {
        float sums[WORK_GROUP_SIZE];
        const float m = mean[wg];
        for (int l = 0; l < WORK_GROUP_SIZE; l++) {
            const size_t i = wg * WORK_GROUP_SIZE * reduction_size + (size_t)l;
            float sum = 0.0f;
            for (size_t j = 0; j < reduction_size; j++) {
                /* K/group_norm.cl:43: (x - mean) * (x - mean), biased (:54) */
                const float d = input[i + WORK_GROUP_SIZE * j] - m;
                sum += d * d;
            }
            sums[l] = sum;
        }
        output[wg] = tree_reduce_64(sums) / (float)(WORK_GROUP_SIZE * reduction_size);
    }
}

void orc_group_norm(const float *input, const float *mean, const float *variance,
                    const float *weight, const float *bias, size_t group_size,
                    size_t channel_size, float epsilon, float *output, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t id = 0; id < n; id++) {
        const size_t group_id = id / group_size;     /* K/group_norm.cl:70 */
        const size_t channel_id = id / channel_size; /* K/group_norm.cl:71 */
        float temp = input[id] - mean[group_id];
        temp /= sqrtf(variance[group_id] + epsilon);
        output[id] = fmaf(temp, weight[channel_id], bias[channel_id]);
    }
}

void orc_layer_norm(const float *input, const float *mean, const float *variance,
                    const float *weight, const float *bias, size_t chunk_size,
                    float epsilon, float *output, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t id = 0; id < n; id++) {
        const size_t chunk_id = id % chunk_size;       /* K/layer_norm.cl:72 */
        const size_t chunk_group_id = id / chunk_size; /* K/layer_norm.cl:73 */
        float temp = input[id] - mean[chunk_group_id];
        temp /= sqrtf(variance[chunk_group_id] + epsilon);
        output[id] = fmaf(temp, weight[chunk_id], bias[chunk_id]);
    }
}

void orc_silu(const float *src, float *dst, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) {
        const float x = src[i];
        float temp = expf(-x); /* K/util.cl:131 */
        temp = 1.0f / (1.0f + temp);
        dst[i] = x * temp;
    }
}

#define ORC_SQRT1_2_F 0.70710678118654752440f /* OpenCL M_SQRT1_2_F */

void orc_gelu(const float *src, float *dst, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) {
        const float x = src[i];
        float temp = x * ORC_SQRT1_2_F; /* K/util.cl:119 */
        temp = 1.0f + erff(temp);
        dst[i] = x * 0.5f * temp;
    }
}

void orc_quick_gelu(const float *src, float *dst, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) {
        const float x = src[i];
        float temp = expf(-(1.702f * x));
        temp = 1.0f / (1.0f + temp);
        dst[i] = x * temp;
    }
}

void orc_gelu_multiply(const float *ab, float *dst, size_t rows, size_t inner) {
#pragma omp parallel for schedule(static)
    for (size_t r = 0; r < rows; r++) {
        for (size_t c = 0; c < inner; c++) {
            const size_t idx = r * inner * 2 + c; /* K/geglu.cl:5-6 */
            const float a = ab[idx];
            const float b = ab[idx + inner];
            float temp = b * ORC_SQRT1_2_F; /* K/geglu.cl:19-21 */
            temp = 1.0f + erff(temp);
            temp = b * 0.5f * temp;
            dst[r * inner + c] = a * temp;
        }
    }
}

void orc_elemwise_add(const float *a, const float *b, float *c, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) c[i] = a[i] + b[i]; /* K/util.cl:11 */
}

void orc_chunkwise_add(const float *a, const float *chunk, float *c, size_t n, size_t chunk_size) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) c[i] = a[i] + chunk[i / chunk_size]; /* K/util.cl:143-147 */
}

void orc_permute3D_0_2_1(const float *src, float *dst, size_t isize, size_t jsize, size_t ksize) {
    /* K/util.cl:47-64: i j k -> i k j */
    for (size_t i = 0; i < isize; i++)
        for (size_t j = 0; j < jsize; j++)
            for (size_t k = 0; k < ksize; k++)
                dst[i * ksize * jsize + k * jsize + j] = src[i * jsize * ksize + j * ksize + k];
}

void orc_timestep_freqs(float *freq, int half, float max_period) {
    for (int i = 0; i < half; i++) /* M/UNetModel.cpp:1950, float overloads throughout */
        freq[i] = expf((-logf(max_period)) * (float)i / (float)half);
}

void orc_timestep_embedding(int64_t timestep, float *out, int dim, float max_period) {
    const int half = dim / 2;
    for (int i = 0; i < half; i++) {
        const float freq = expf((-logf(max_period)) * (float)i / (float)half);
        const float arg = (float)timestep * freq;
        out[i] = cosf(arg);        /* [cos | sin] order, M/UNetModel.cpp:1952-1953 */
        out[i + half] = sinf(arg);
    }
}

int orc_ddim_timesteps(int ddim_num_steps, int *out, int cap) {
    const int ddpm_num_time_steps = 1000; /* M/DDIMSampler.cpp:13 */
    if (ddim_num_steps <= 0 || ddim_num_steps > ddpm_num_time_steps) return -1;
    const int c = ddpm_num_time_steps / ddim_num_steps;
    int count = 0;
    for (int i = 0; i < ddpm_num_time_steps; i += c) {
        if (count < cap) out[count] = i + 1;
        count++;
    }
    return count;
}

/* ------------------------------------------------------------------ */
/* host-object drivers                                                 */
/* ------------------------------------------------------------------ */
int orc_groupnorm_forward(const float *x, float *y, const float *weight, const float *bias,
                          size_t batch, size_t channels, size_t hw, size_t groups, float eps,
                          int silu) {
    const size_t input_size = channels * hw; /* one sample: the reference's whole buffer */
    if (groups == 0 || channels == 0 || input_size % channels != 0) return -1;
    const size_t group_size = input_size / groups;            /* M/nn/GroupNorm.cpp:80 */
    const size_t reduction_size = group_size / WORK_GROUP_SIZE; /* :81 */
    if (group_size % WORK_GROUP_SIZE != 0 || reduction_size == 0) return -1; /* :89-93 */
    const size_t channel_size = input_size / channels;        /* :130 */
    float mean[groups], var[groups];
    for (size_t b = 0; b < batch; b++) {
        const float *xs = x + b * input_size;
        float *ys = y + b * input_size;
        orc_local_reduction_mean(xs, mean, groups, reduction_size);
        orc_local_reduction_variance(xs, mean, var, groups, reduction_size);
        orc_group_norm(xs, mean, var, weight, bias, group_size, channel_size, eps, ys,
                       input_size);
        if (silu) orc_silu(ys, ys, input_size); /* in place, M/nn/ResBlock.cpp:136-142 */
    }
    return 0;
}

int orc_layernorm_forward(const float *x, float *y, const float *weight, const float *bias,
                          size_t rows, size_t dim, float eps) {
    if (dim == 0 || dim % WORK_GROUP_SIZE != 0) return -1; /* M/nn/LayerNorm.cpp:61 */
    const size_t reduction_size = dim / WORK_GROUP_SIZE;   /* :93 */
    float *mean = (float *)__builtin_malloc(sizeof(float) * (rows ? rows : 1));
    float *var = (float *)__builtin_malloc(sizeof(float) * (rows ? rows : 1));
    if (!mean || !var) {
        __builtin_free(mean);
        __builtin_free(var);
        return -2;
    }
    orc_local_reduction_mean(x, mean, rows, reduction_size);
    orc_local_reduction_variance(x, mean, var, rows, reduction_size);
    orc_layer_norm(x, mean, var, weight, bias, dim, eps, y, rows * dim);
    __builtin_free(mean);
    __builtin_free(var);
    return 0;
}

/* ------------------------------------------------------------------ */
/* float64 textbook versions                                           */
/* ------------------------------------------------------------------ */
void orc64_groupnorm(const float *x, double *y, const float *weight, const float *bias,
                     size_t batch, size_t channels, size_t hw, size_t groups, double eps,
                     int silu) {
    const size_t cpg = channels / groups;
    const size_t gsz = cpg * hw;
#pragma omp parallel for schedule(static)
    for (size_t u = 0; u < batch * groups; u++) {
        const size_t b = u / groups, g = u % groups;
        const float *xs = x + (b * channels + g * cpg) * hw;
        double *ys = y + (b * channels + g * cpg) * hw;
        double s = 0.0;
        for (size_t i = 0; i < gsz; i++) s += xs[i];
        const double m = s / (double)gsz;
        double q = 0.0;
        for (size_t i = 0; i < gsz; i++) q += (xs[i] - m) * (xs[i] - m);
        const double rstd = 1.0 / sqrt(q / (double)gsz + eps);
        for (size_t i = 0; i < gsz; i++) {
            const size_t c = g * cpg + i / hw;
            double v = (xs[i] - m) * rstd * (double)weight[c] + (double)bias[c];
            if (silu) v = v / (1.0 + exp(-v));
            ys[i] = v;
        }
    }
}

void orc64_layernorm(const float *x, double *y, const float *weight, const float *bias,
                     size_t rows, size_t dim, double eps) {
#pragma omp parallel for schedule(static)
    for (size_t r = 0; r < rows; r++) {
        const float *xs = x + r * dim;
        double s = 0.0;
        for (size_t i = 0; i < dim; i++) s += xs[i];
        const double m = s / (double)dim;
        double q = 0.0;
        for (size_t i = 0; i < dim; i++) q += (xs[i] - m) * (xs[i] - m);
        const double rstd = 1.0 / sqrt(q / (double)dim + eps);
        for (size_t i = 0; i < dim; i++)
            y[r * dim + i] = (xs[i] - m) * rstd * (double)weight[i] + (double)bias[i];
    }
}

void orc64_silu(const float *x, double *y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = (double)x[i] / (1.0 + exp(-(double)x[i]));
}

void orc64_gelu(const float *x, double *y, size_t n) {
    for (size_t i = 0; i < n; i++)
        y[i] = 0.5 * (double)x[i] * erfc(-(double)x[i] * 0.70710678118654752440);
}

void orc64_quick_gelu(const float *x, double *y, size_t n) {
    for (size_t i = 0; i < n; i++)
        y[i] = (double)x[i] / (1.0 + exp(-(double)1.702f * (double)x[i]));
}

void orc64_geglu(const float *ab, double *y, size_t rows, size_t inner) {
    for (size_t r = 0; r < rows; r++)
        for (size_t c = 0; c < inner; c++) {
            const double a = ab[r * 2 * inner + c];
            const double b = ab[r * 2 * inner + inner + c];
            y[r * inner + c] = a * 0.5 * b * erfc(-b * 0.70710678118654752440);
        }
}

void orc64_timestep_embedding(int64_t timestep, double *out, int dim, double max_period) {
    const int half = dim / 2;
    for (int i = 0; i < half; i++) {
        const double freq = exp(-log(max_period) * (double)i / (double)half);
        out[i] = cos((double)timestep * freq);
        out[i + half] = sin((double)timestep * freq);
    }
}

/* ------------------------------------------------------------------ */
/* neighbours of the path: embedding Linear, row softmax, DDIM schedule */
/* ------------------------------------------------------------------ */

/* K/linear.cl:345-430 (tile_reg_n_vector_linear, the variant LINEAR_KERNEL_VERSION 4
 * of M/setting.h:8 selects, M/nn/Linear.cpp:244-289): C[i,j] = sum_k A[i,k]*B[j,k],
 * one float accumulator per output, k ascending, bias added last. */
void orc_linear(const float *a, const float *w, const float *bias, float *c, size_t m, size_t n,
                size_t k) {
#pragma omp parallel for collapse(2) schedule(static)
    for (size_t i = 0; i < m; i++)
        for (size_t j = 0; j < n; j++) {
            float acc = 0.0f;
            for (size_t kk = 0; kk < k; kk++) acc += a[i * k + kk] * w[j * k + kk];
            if (bias != NULL) acc += bias[j];
            c[i * n + j] = acc;
        }
}

void orc64_linear(const float *a, const float *w, const float *bias, double *c, size_t m, size_t n,
                  size_t k) {
    for (size_t i = 0; i < m; i++)
        for (size_t j = 0; j < n; j++) {
            double acc = 0.0;
            for (size_t kk = 0; kk < k; kk++) acc += (double)a[i * k + kk] * (double)w[j * k + kk];
            if (bias != NULL) acc += (double)bias[j];
            c[i * n + j] = acc;
        }
}

/* K/util.cl:150-187: one workgroup of local_size lanes per chunk; lane-strided
 * partial sums of exp(x) (no maximum is subtracted), the tree of :172-180 with its
 * odd-size bookkeeping, then exp(x) / total.  The call sites use 64 lanes
 * (M/nn/CrossAttention.cpp:362-377, M/nn/AttnBlock.cpp:196-206). */
void orc_softmax(const float *input, float *output, size_t rows, size_t chunk_size,
                 size_t local_size) {
#pragma omp parallel for schedule(static)
    for (size_t wg = 0; wg < rows; wg++) {
        const float *in = input + wg * chunk_size;
        float *out = output + wg * chunk_size;
        float sums[1024];
        float cache_small[4096];
        float *cache = chunk_size <= 4096 ? cache_small : (float *)malloc(chunk_size * sizeof(float));
        for (size_t lid = 0; lid < local_size; lid++) {
            float sum = 0.0f;
            for (size_t index = lid; index < chunk_size; index += local_size) {
                const float e = expf(in[index]);
                sum += e;
                cache[index] = e;
            }
            sums[lid] = sum;
        }
        size_t remainder = local_size % 2;
        for (size_t offset = local_size / 2; offset > 0; offset /= 2) {
            for (size_t lid = 0; lid < offset; lid++)
                sums[lid + remainder] += sums[lid + offset + remainder];
            offset += remainder;
            remainder = offset % 2;
        }
        for (size_t index = 0; index < chunk_size; index++) out[index] = cache[index] / sums[0];
        if (cache != cache_small) free(cache);
    }
}

/* textbook softmax with the row maximum subtracted, float64 */
void orc64_softmax(const float *input, double *output, size_t rows, size_t chunk_size) {
    for (size_t r = 0; r < rows; r++) {
        const float *in = input + r * chunk_size;
        double mx = -INFINITY, total = 0.0;
        for (size_t i = 0; i < chunk_size; i++) mx = in[i] > mx ? in[i] : mx;
        for (size_t i = 0; i < chunk_size; i++) total += exp((double)in[i] - mx);
        for (size_t i = 0; i < chunk_size; i++)
            output[r * chunk_size + i] = exp((double)in[i] - mx) / total;
    }
}

/* M/DDIMSampler.cpp:18-39: betas = linspace(sqrt(0.00085), sqrt(0.0120), 1000)^2 in
 * double (linspace at :139-153), alphas = 1 - beta, running product in double,
 * stored as float. */
void orc_alphas_cumprod(float *out) {
    const int steps = 1000;
    const double start = sqrt(0.00085), end = sqrt(0.0120);
    const double step_size = (end - start) / (double)(steps - 1);
    double acc = 1.0;
    for (int i = 0; i < steps; i++) {
        double beta = start + (double)i * step_size;
        beta = beta * beta;
        const double alpha = 1.0f - beta;
        acc = i == 0 ? alpha : acc * alpha;
        out[i] = (float)acc;
    }
}

/* M/DDIMSampler.cpp:60-76 with make_schedule (:123-137): alphas[i] = cumprod[ts[i]],
 * alphas_prev = {cumprod[0], cumprod[ts[0]], ...}, sqrt(1 - alphas).  Returns the
 * count, -1 for steps outside [1, 1000], -2 when the list reaches 1000 (the
 * reference would index one past its 1000-entry table). */
int orc_ddim_schedule(int ddim_num_steps, int *timesteps, float *alphas, float *alphas_prev,
                      float *sqrt_one_minus_alphas, int cap) {
    int ts[1001];
    const int count = orc_ddim_timesteps(ddim_num_steps, ts, 1001);
    if (count < 0) return -1;
    if (ts[count - 1] >= 1000) return -2;
    float cumprod[1000];
    orc_alphas_cumprod(cumprod);
    for (int i = 0; i < count && i < cap; i++) {
        timesteps[i] = ts[i];
        alphas[i] = cumprod[ts[i]];
        alphas_prev[i] = i == 0 ? cumprod[0] : cumprod[ts[i - 1]];
        sqrt_one_minus_alphas[i] = sqrtf(1.0f - alphas[i]);
    }
    return count;
}

/* M/DDIMSampler.cpp:94-121 (eta = 0): three float loops; sqrt on float values
 * (the reference builds with libc++, whose ::sqrt(float) is the float overload). */
void orc_ddim_update(const float *x, const float *e_t, float *x_prev, size_t n, float a_t,
                     float a_prev, float sqrt_one_minus_at) {
    for (size_t i = 0; i < n; i++) {
        const float pred_x0 = (x[i] - sqrt_one_minus_at * e_t[i]) / sqrtf(a_t);
        const float dir_xt = sqrtf(1.0f - a_prev) * e_t[i];
        x_prev[i] = sqrtf(a_prev) * pred_x0 + dir_xt;
    }
}

void orc64_ddim_update(const float *x, const float *e_t, double *x_prev, size_t n, double a_t,
                       double a_prev) {
    for (size_t i = 0; i < n; i++) {
        const double pred_x0 = ((double)x[i] - sqrt(1.0 - a_t) * (double)e_t[i]) / sqrt(a_t);
        x_prev[i] = sqrt(a_prev) * pred_x0 + sqrt(1.0 - a_prev) * (double)e_t[i];
    }
}

/* ------------------------------------------------------------------ */
int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void orc_set_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}
