// Host utilities of the layer objects: the weight loader, the golden-file comparison and
// event timing, mirroring namespace util of the reference (M/util.h:16-36).
#pragma once

#include <hip/hip_runtime_api.h>

#include <string>
#include <vector>

#include "DeviceBuffer.h"
#include "npy.h"

namespace msd {
namespace util {

// Directory prepended to every weight / fixture file name.  The reference hard-codes
// "/sdcard/Android/media/com.example.myopencl/" (M/util.cpp:15); here it comes from
// setMediaPath(), else the MSD_MEDIA_PATH environment variable, else "./".
void setMediaPath(const std::string &dir);
std::string mediaPath();

// Host copy of an .npy file under the media path (M/util.cpp:97-101).
npy::Array load_npy_file(const std::string &filename);

// Device copy (float32) of an .npy file under the media path; *num_vals receives the element
// count (M/util.cpp:103-147).  Throws std::runtime_error for file / format / HIP failures.
DeviceBuffer load_npy_file(const std::string &filename, size_t *num_vals, hipStream_t stream);

// Uploads host floats into a new device buffer, converting to `dtype` storage.
DeviceBuffer upload(const std::vector<float> &data, DType dtype, hipStream_t stream);
// Downloads a device buffer as floats (fp16 storage is widened).
std::vector<float> download(const DeviceBuffer &buffer, hipStream_t stream);

// Result of comparing a buffer with a golden .npy file: the figures the reference logs
// (max abs diff, number of elements that differ at all, index of the largest diff).
struct TestResult {
    bool size_matches = false;
    float max_diff = 0.0f;
    size_t num_wrong = 0;
    size_t max_id = 0;
};
// Reads the buffer back, loads `filename` (relative to the media path) and compares element
// by element with != exactly as util::testBuffer does (M/util.cpp:149-201); prints the same
// one-line summary to stderr.
TestResult testBuffer(hipStream_t stream, const DeviceBuffer &buffer, const char *filename);
TestResult testBuffer(const std::vector<float> &result, const char *filename);

// Milliseconds between two recorded events, printed as "<message>, <ms>" like
// util::printEventTime (M/util.cpp:203-215).  Returns the value (negative on error).
float printEventTime(const std::string &message, hipEvent_t start, hipEvent_t stop);

// Per-launch timing rows like the reference's `#define DEBUG 1` blocks
// (M/nn/GroupNorm.cpp:147-162, M/nn/LayerNorm.cpp:144-154): switched on at run time by
// setDebugTiming(true) or the MSD_DEBUG_TIMING=1 environment variable.  A LaunchTimer
// brackets one launch with two events; finish() waits for it and prints
// "<message>, <ms>" through printEventTime.  With timing off both calls do nothing.
void setDebugTiming(bool on);
bool debugTiming();
class LaunchTimer {
public:
    explicit LaunchTimer(hipStream_t stream);
    ~LaunchTimer();
    LaunchTimer(const LaunchTimer &) = delete;
    LaunchTimer &operator=(const LaunchTimer &) = delete;
    // Returns the milliseconds (negative when timing is off or an event call failed).
    float finish(const std::string &message);

private:
    hipStream_t stream_;
    hipEvent_t start_ = nullptr;
    hipEvent_t stop_ = nullptr;
};

}  // namespace util
}  // namespace msd
