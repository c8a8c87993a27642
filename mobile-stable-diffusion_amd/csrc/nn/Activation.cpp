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

}  // namespace msd
