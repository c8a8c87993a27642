#include "Activation.h"

#include <stdexcept>

namespace msd {
namespace {
typedef int (*act_fn)(const void *, void *, size_t, int, void *);

int run(act_fn fn, hipStream_t stream, const DeviceBuffer &src, DeviceBuffer &dst) {
    if (dst.bytes() != src.bytes() || dst.dtype() != src.dtype())
        throw std::runtime_error("dst size / type != src size / type");
    return fn(src.ptr(), dst.ptr(), src.count(), (int)src.dtype(), stream);
}
}  // namespace

int silu(hipStream_t stream, const DeviceBuffer &src, DeviceBuffer &dst) {
    return run(msd_silu, stream, src, dst);
}
int gelu(hipStream_t stream, const DeviceBuffer &src, DeviceBuffer &dst) {
    return run(msd_gelu, stream, src, dst);
}
int quick_gelu(hipStream_t stream, const DeviceBuffer &src, DeviceBuffer &dst) {
    return run(msd_quick_gelu, stream, src, dst);
}

int elemwise_add(hipStream_t stream, const DeviceBuffer &a, const DeviceBuffer &b, DeviceBuffer &c) {
    if (b.bytes() != a.bytes() || c.bytes() != a.bytes() || b.dtype() != a.dtype() || c.dtype() != a.dtype())
        throw std::runtime_error("operand sizes / types differ");
    return msd_elemwise_add(a.ptr(), b.ptr(), c.ptr(), a.count(), (int)a.dtype(), stream);
}

int chunkwise_add(hipStream_t stream, const DeviceBuffer &a, const DeviceBuffer &chunk, DeviceBuffer &c,
                  size_t chunk_size) {
    if (c.bytes() != a.bytes() || c.dtype() != a.dtype() || chunk.dtype() != a.dtype() || chunk_size == 0 ||
        a.count() % chunk_size != 0 || chunk.count() != a.count() / chunk_size)
        throw std::runtime_error("chunk size does not match the operand");
    return msd_chunkwise_add(a.ptr(), chunk.ptr(), c.ptr(), a.count(), chunk_size, (int)a.dtype(), stream);
}

int permute3D_0_2_1(hipStream_t stream, const DeviceBuffer &src, DeviceBuffer &dst, size_t isize,
                    size_t jsize, size_t ksize) {
    if (dst.bytes() != src.bytes() || dst.dtype() != src.dtype() || src.count() != isize * jsize * ksize)
        throw std::runtime_error("buffer size does not match i * j * k");
    return msd_permute_0_2_1(src.ptr(), dst.ptr(), isize, jsize, ksize, (int)src.dtype(), stream);
}

int softmax(hipStream_t stream, const DeviceBuffer &src, DeviceBuffer &dst, size_t chunkSize, bool stable) {
    if (dst.bytes() != src.bytes() || dst.dtype() != src.dtype())
        throw std::runtime_error("dst size / type != src size / type");
    if (chunkSize == 0 || src.count() % chunkSize != 0)
        throw std::runtime_error("element count % chunkSize != 0");
    return msd_softmax(src.ptr(), dst.ptr(), src.count() / chunkSize, chunkSize, stable ? 1 : 0,
                       (int)src.dtype(), stream);
}

}  // namespace msd
