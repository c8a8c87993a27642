// Plain-C handles over the C++ layer objects, for callers that cannot bind C++ (the tests
// drive the objects through these with ctypes; a JNI or cgo stub would bind the same
// functions).  Every function returns 0 on success; a negative value means a C++ exception
// was caught and msdnn_last_error() holds its text (the layer objects throw
// std::runtime_error where the reference does); a positive value is a hipError_t.
#include <hip/hip_runtime.h>

#include <cstring>
#include <exception>
#include <string>

#include "Activation.h"
#include "GEGLU.h"
#include "DDIMSampler.h"
#include "GroupNorm.h"
#include "LayerNorm.h"
#include "Linear.h"
#include "TimestepEmbedding.h"
#include "UNetNormActStep.h"
#include "util.h"

using namespace msd;

namespace {
thread_local std::string g_last_error;

template <typename F>
int guarded(F f) {
    try {
        return f();
    } catch (const std::exception &e) {
        g_last_error = e.what();
        return -1;
    } catch (...) {
        g_last_error = "unknown exception";
        return -1;
    }
}

DeviceBuffer wrap(void *p, size_t bytes, int dtype) {
    return DeviceBuffer(p, bytes, dtype == MSD_DTYPE_F16 ? DType::F16 : DType::F32);
}
}  // namespace

extern "C" {

const char *msdnn_last_error(void) { return g_last_error.c_str(); }

void msdnn_set_media_path(const char *dir) { util::setMediaPath(dir ? dir : ""); }

// per-launch timing rows on stderr (the reference's DEBUG blocks); 0 switches them off
void msdnn_set_debug_timing(int on) { util::setDebugTiming(on != 0); }

// ---- npy (host only)
int msdnn_npy_load(const char *name, float *out, size_t cap, size_t *num_vals, size_t *ndim) {
    return guarded([&] {
        const npy::Array a = util::load_npy_file(name);
        if (num_vals) *num_vals = a.num_vals();
        if (ndim) *ndim = a.shape.size();
        if (out) memcpy(out, a.data.data(), sizeof(float) * (a.num_vals() < cap ? a.num_vals() : cap));
        return 0;
    });
}
int msdnn_npy_save(const char *path, const float *data, size_t n) {
    return guarded([&] {
        npy::save(path, {n}, data);
        return 0;
    });
}

// ---- GroupNorm
void *msdnn_groupnorm_create(void *stream, size_t num_groups, size_t num_channels, float eps,
                             const char *weight_name, const char *bias_name, size_t batch, int fuse_silu) {
    GroupNorm *g = nullptr;
    guarded([&] {
        g = new GroupNorm(static_cast<hipStream_t>(stream), num_groups, num_channels, eps, weight_name,
                          bias_name, batch, fuse_silu != 0);
        return 0;
    });
    return g;
}
int msdnn_groupnorm_init(void *h) {
    return guarded([&] {
        static_cast<GroupNorm *>(h)->init();
        return 0;
    });
}
int msdnn_groupnorm_check(void *h, size_t input_bytes, int dtype) {
    return guarded([&] {
        static_cast<GroupNorm *>(h)->checkInput(input_bytes, dtype == MSD_DTYPE_F16 ? DType::F16 : DType::F32);
        return 0;
    });
}
int msdnn_groupnorm_forward(void *h, void *in, void *out, size_t bytes, int dtype) {
    return guarded([&] {
        DeviceBuffer i = wrap(in, bytes, dtype), o = wrap(out, bytes, dtype);
        return static_cast<GroupNorm *>(h)->forward(i, o);
    });
}
int msdnn_groupnorm_forward_chunk(void *h, void *in, void *chunk, size_t chunk_bytes, void *out, size_t bytes,
                                  int dtype) {
    return guarded([&] {
        DeviceBuffer i = wrap(in, bytes, dtype), c = wrap(chunk, chunk_bytes, dtype), o = wrap(out, bytes, dtype);
        return static_cast<GroupNorm *>(h)->forward(i, c, o);
    });
}
int msdnn_groupnorm_forward_tokens(void *h, void *in, void *out, size_t bytes, int dtype) {
    return guarded([&] {
        DeviceBuffer i = wrap(in, bytes, dtype), o = wrap(out, bytes, dtype);
        return static_cast<GroupNorm *>(h)->forwardTokens(i, o);
    });
}
void msdnn_groupnorm_destroy(void *h) { delete static_cast<GroupNorm *>(h); }

// ---- LayerNorm
void *msdnn_layernorm_create(void *stream, size_t dim, const char *weight_name, const char *bias_name,
                             float eps) {
    LayerNorm *l = nullptr;
    guarded([&] {
        l = new LayerNorm(static_cast<hipStream_t>(stream), dim, weight_name, bias_name, eps);
        return 0;
    });
    return l;
}
int msdnn_layernorm_init(void *h) {
    return guarded([&] {
        static_cast<LayerNorm *>(h)->init();
        return 0;
    });
}
int msdnn_layernorm_check(void *h, size_t input_bytes, int dtype) {
    return guarded([&] {
        static_cast<LayerNorm *>(h)->checkInput(input_bytes, dtype == MSD_DTYPE_F16 ? DType::F16 : DType::F32);
        return 0;
    });
}
int msdnn_layernorm_forward(void *h, void *in, void *out, size_t bytes, int dtype) {
    return guarded([&] {
        DeviceBuffer i = wrap(in, bytes, dtype), o = wrap(out, bytes, dtype);
        return static_cast<LayerNorm *>(h)->forward(i, o);
    });
}
int msdnn_layernorm_forward_add(void *h, void *a, void *b, void *sum, void *out, size_t bytes, int dtype) {
    return guarded([&] {
        DeviceBuffer ab = wrap(a, bytes, dtype), bb = wrap(b, bytes, dtype), sb = wrap(sum, bytes, dtype),
                     ob = wrap(out, bytes, dtype);
        return static_cast<LayerNorm *>(h)->forwardAdd(ab, bb, sb, ob);
    });
}
void msdnn_layernorm_destroy(void *h) { delete static_cast<LayerNorm *>(h); }

// ---- GEGLU
void *msdnn_geglu_create(void *stream, size_t in_features, size_t out_features) {
    return new GEGLU(static_cast<hipStream_t>(stream), in_features, out_features);
}
int msdnn_geglu_weight_shape(void *h, size_t *rows, size_t *cols) {
    *rows = static_cast<GEGLU *>(h)->weightShape[0];
    *cols = static_cast<GEGLU *>(h)->weightShape[1];
    return 0;
}
int msdnn_geglu_check(void *h, size_t in_bytes, size_t out_bytes, int dtype) {
    return guarded([&] {
        static_cast<GEGLU *>(h)->checkInput(in_bytes, out_bytes, dtype == MSD_DTYPE_F16 ? DType::F16 : DType::F32);
        return 0;
    });
}
int msdnn_geglu_forward(void *h, void *in, size_t in_bytes, void *out, size_t out_bytes, int dtype) {
    return guarded([&] {
        DeviceBuffer i = wrap(in, in_bytes, dtype), o = wrap(out, out_bytes, dtype);
        return static_cast<GEGLU *>(h)->forward(i, o);
    });
}
void msdnn_geglu_destroy(void *h) { delete static_cast<GEGLU *>(h); }

// ---- activations: op 0 silu, 1 gelu, 2 quick_gelu
int msdnn_activation(void *stream, int op, void *src, void *dst, size_t bytes, int dtype) {
    return guarded([&] {
        DeviceBuffer s = wrap(src, bytes, dtype), d = wrap(dst, bytes, dtype);
        hipStream_t st = static_cast<hipStream_t>(stream);
        return op == 0 ? silu(st, s, d) : op == 1 ? gelu(st, s, d) : quick_gelu(st, s, d);
    });
}

// ---- timestep embedding: writes batch*dim floats to host memory `out`
int msdnn_timestep_embedding(void *stream, const long *timesteps, size_t batch, float *out) {
    return guarded([&] {
        hipStream_t st = static_cast<hipStream_t>(stream);
        DeviceBuffer e = createTimestepEmbedding(st, std::vector<long>(timesteps, timesteps + batch));
        const std::vector<float> host = util::download(e, st);
        memcpy(out, host.data(), host.size() * sizeof(float));
        return 0;
    });
}
int msdnn_ddim_timesteps(int steps, int *out, int cap) {
    int n = 0;
    const int rc = guarded([&] {
        const std::vector<int> t = ddimTimesteps(steps);
        n = (int)t.size();
        for (int i = 0; i < n && i < cap; i++) out[i] = t[(size_t)i];
        return 0;
    });
    return rc < 0 ? rc : n;
}

// ---- Linear on embedding rows; weights from .npy names (init) or from host arrays (init_from)
void *msdnn_linear_create(void *stream, size_t in_features, size_t out_features, const char *weight_name,
                          const char *bias_name, int dtype) {
    Linear *l = nullptr;
    guarded([&] {
        l = new Linear(static_cast<hipStream_t>(stream), in_features, out_features, weight_name ? weight_name : "",
                       bias_name ? bias_name : "", dtype == MSD_DTYPE_F16 ? DType::F16 : DType::F32);
        return 0;
    });
    return l;
}
int msdnn_linear_init(void *h) {
    return guarded([&] {
        static_cast<Linear *>(h)->init();
        return 0;
    });
}
int msdnn_linear_init_from(void *h, const float *weight, size_t weight_count, const float *bias,
                           size_t bias_count) {
    return guarded([&] {
        static_cast<Linear *>(h)->init(std::vector<float>(weight, weight + weight_count),
                                       bias ? std::vector<float>(bias, bias + bias_count) : std::vector<float>());
        return 0;
    });
}
int msdnn_linear_forward(void *h, void *in, size_t in_bytes, void *out, size_t out_bytes, int dtype,
                         int silu_on_input, int silu_on_output) {
    return guarded([&] {
        DeviceBuffer i = wrap(in, in_bytes, dtype), o = wrap(out, out_bytes, dtype);
        return static_cast<Linear *>(h)->forwardSilu(i, o, silu_on_input != 0, silu_on_output != 0);
    });
}
// `count` Linear handles on the same input rows in one launch; outs / out_bytes are host arrays
int msdnn_linear_forward_grouped(void *const *hs, size_t count, void *in, size_t in_bytes, void *const *outs,
                                 const size_t *out_bytes, int dtype, int silu_on_input, int silu_on_output) {
    return guarded([&] {
        std::vector<Linear *> layers(count);
        std::vector<DeviceBuffer> outputs;
        for (size_t i = 0; i < count; i++) {
            layers[i] = static_cast<Linear *>(hs[i]);
            outputs.push_back(wrap(outs[i], out_bytes[i], dtype));
        }
        const DeviceBuffer input = wrap(in, in_bytes, dtype);
        return Linear::forwardSiluGrouped(layers, input, outputs, silu_on_input != 0, silu_on_output != 0);
    });
}
void msdnn_linear_destroy(void *h) { delete static_cast<Linear *>(h); }

// ---- row softmax
int msdnn_softmax(void *stream, void *src, void *dst, size_t bytes, int dtype, size_t chunk_size, int stable) {
    return guarded([&] {
        DeviceBuffer s = wrap(src, bytes, dtype), d = wrap(dst, bytes, dtype);
        return softmax(static_cast<hipStream_t>(stream), s, d, chunk_size, stable != 0);
    });
}

// ---- DDIM sampler.  The noise model is a C callback: model(x, t, e_t, bytes, user) fills e_t for
// latent x on the sampler's stream and returns 0.  x_T (device, `bytes` long) is not modified;
// the final latent is copied to `out` (device, same size).
typedef int (*msdnn_model_fn)(void *x, int t, void *e_t, size_t bytes, void *user);
int msdnn_ddim_sample(void *stream, void *x_T, size_t bytes, int dtype, int steps, msdnn_model_fn model,
                      void *user, void *out) {
    return guarded([&] {
        hipStream_t st = static_cast<hipStream_t>(stream);
        DDIMSampler sampler(st, [&](const DeviceBuffer &x, int t, const DeviceBuffer &, DeviceBuffer &e_t) {
            return model(x.ptr(), t, e_t.ptr(), x.bytes(), user);
        });
        DeviceBuffer start = wrap(x_T, bytes, dtype), none;
        const int shape[3] = {0, 0, 0};
        DeviceBuffer img = sampler.sample(&start, steps, shape, none);
        return (int)hipMemcpy(out, img.ptr(), bytes, hipMemcpyDeviceToDevice);
    });
}
// make_schedule through the sampler object: alphas / alphas_prev for a timestep list
int msdnn_ddim_make_schedule(const int *timesteps, int count, float *alphas, float *alphas_prev) {
    return guarded([&] {
        DDIMSampler sampler(nullptr, DDIMSampler::ApplyModel());
        const auto s = sampler.make_schedule(std::vector<int>(timesteps, timesteps + count));
        for (int i = 0; i < count; i++) {
            alphas[i] = s.first[(size_t)i];
            alphas_prev[i] = s.second[(size_t)i];
        }
        return 0;
    });
}

// ---- golden-file comparison (util::testBuffer)
int msdnn_test_buffer(void *stream, void *ptr, size_t bytes, int dtype, const char *golden, float *max_diff,
                      size_t *num_wrong) {
    return guarded([&] {
        const util::TestResult r =
            util::testBuffer(static_cast<hipStream_t>(stream), wrap(ptr, bytes, dtype), golden);
        if (max_diff) *max_diff = r.max_diff;
        if (num_wrong) *num_wrong = r.num_wrong;
        return r.size_matches ? 0 : -2;
    });
}

// ---- one UNet step of the path
void *msdnn_step_create(void *stream, size_t batch, int dtype, int keep_inputs) {
    UNetNormActStep *s = nullptr;
    guarded([&] {
        s = new UNetNormActStep(static_cast<hipStream_t>(stream), batch,
                                dtype == MSD_DTYPE_F16 ? DType::F16 : DType::F32, 5001, keep_inputs != 0);
        return 0;
    });
    return s;
}
// what launch i works on: kind 0 GroupNorm+SiLU {channels, hw}, 1 LayerNorm {rows, dim},
// 2 GEGLU {rows, inner}, 3 SiLU {n, 0}
size_t msdnn_step_num_ops(void *h) { return static_cast<UNetNormActStep *>(h)->numOps(); }
int msdnn_step_op_info(void *h, size_t i, int *kind, size_t *dims, int *in_place) {
    return guarded([&] {
        const UNetNormActStep::OpInfo info = static_cast<UNetNormActStep *>(h)->opInfo(i);
        *kind = info.kind;
        dims[0] = info.dims[0];
        dims[1] = info.dims[1];
        *in_place = info.in_place ? 1 : 0;
        return 0;
    });
}
// which: 0 input of launch i, 1 output of launch i, 2 the timestep embedding (i ignored);
// writes at most cap floats, *count receives the element count
int msdnn_step_download(void *h, size_t i, int which, float *dst, size_t cap, size_t *count) {
    return guarded([&] {
        UNetNormActStep *s = static_cast<UNetNormActStep *>(h);
        const std::vector<float> v = which == 0 ? s->downloadInput(i) : which == 1 ? s->downloadOutput(i)
                                                                                    : s->downloadEmbedding();
        if (count) *count = v.size();
        if (dst) memcpy(dst, v.data(), sizeof(float) * (v.size() < cap ? v.size() : cap));
        return 0;
    });
}
int msdnn_step_affine(void *h, size_t i, float *gamma, float *beta, size_t cap) {
    return guarded([&] {
        UNetNormActStep *s = static_cast<UNetNormActStep *>(h);
        const std::vector<float> &g = s->weight(i), &b = s->bias(i);
        if (g.size() > cap || b.size() > cap) throw std::runtime_error("msdnn_step_affine: buffer too small");
        memcpy(gamma, g.data(), sizeof(float) * g.size());
        memcpy(beta, b.data(), sizeof(float) * b.size());
        return (int)g.size();
    });
}
int msdnn_step_restore(void *h) {
    return guarded([&] { return static_cast<UNetNormActStep *>(h)->restoreInputs(); });
}
size_t msdnn_step_bytes(void *h) { return static_cast<UNetNormActStep *>(h)->bytesPerStep(); }
size_t msdnn_step_launches(void *h) { return static_cast<UNetNormActStep *>(h)->launchesPerStep(); }
// runs `steps` steps; graph != 0 replays one captured HIP graph per step
int msdnn_step_run(void *h, int steps, int graph, const long *timesteps, size_t batch) {
    return guarded([&] {
        UNetNormActStep *s = static_cast<UNetNormActStep *>(h);
        const std::vector<long> t(timesteps, timesteps + batch);
        int rc = 0;
        if (graph) s->setTimesteps(t);
        for (int i = 0; i < steps && rc == 0; i++) rc = graph ? s->forwardGraph() : s->forward(t);
        return rc;
    });
}
void msdnn_step_destroy(void *h) { delete static_cast<UNetNormActStep *>(h); }

}  // extern "C"
