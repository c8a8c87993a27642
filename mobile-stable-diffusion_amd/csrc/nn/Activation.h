// Elementwise activations.  In the reference these are not objects: a caller sets the two
// arguments of utilKernel->silu / utilKernel->gelu and enqueues it over the element count
// (M/nn/ResBlock.cpp:136-142, M/nn/ResidualAttentionBlock.cpp:146-153).  The equivalents
// take source and destination buffers (the same buffer for the in-place call sites).
#pragma once

#include <hip/hip_runtime_api.h>

#include "DeviceBuffer.h"

namespace msd {

// Each returns 0 or a hipError_t value and throws std::runtime_error when dst and src differ
// in size or storage type.
int silu(hipStream_t stream, const DeviceBuffer &src, DeviceBuffer &dst);        // K/util.cl:124-134
int gelu(hipStream_t stream, const DeviceBuffer &src, DeviceBuffer &dst);        // K/util.cl:104-122
int quick_gelu(hipStream_t stream, const DeviceBuffer &src, DeviceBuffer &dst);  // x*sigmoid(1.702x)

// The two additions of the reference's utility kernels, for call sites that are not fused into
// a norm: c = a + b (K/util.cl:1-12) and c[i] = a[i] + chunk[i / chunk_size] (K/util.cl:136-148).
int elemwise_add(hipStream_t stream, const DeviceBuffer &a, const DeviceBuffer &b, DeviceBuffer &c);
int chunkwise_add(hipStream_t stream, const DeviceBuffer &a, const DeviceBuffer &chunk, DeviceBuffer &c,
                  size_t chunk_size);

// dst[i, k, j] = src[i, j, k]: utilKernel->permute3D_0_2_1 (K/util.cl:47-64), enqueued by
// SpatialTransformer::forward with global size {i, j, k} (M/nn/SpatialTransformer.cpp:136-139).
int permute3D_0_2_1(hipStream_t stream, const DeviceBuffer &src, DeviceBuffer &dst, size_t isize,
                    size_t jsize, size_t ksize);

// Row softmax in chunks of chunkSize elements: utilKernel->softmax (K/util.cl:150-187) as the
// attention blocks enqueue it, in place, one workgroup per chunk
// (M/nn/CrossAttention.cpp:362-377, M/nn/AttnBlock.cpp:196-206).  stable = false is that
// kernel's exp(x) / sum; true subtracts the chunk maximum first.  Throws std::runtime_error
// when the element count is not a multiple of chunkSize.
int softmax(hipStream_t stream, const DeviceBuffer &src, DeviceBuffer &dst, size_t chunkSize,
            bool stable = false);

}  // namespace msd
