// Minimal reader / writer for NPY files holding little-endian float32 in C order: the
// format of every weight file the reference loads (M/util.cpp:103-147 through
// cnpy::parse_npy_header, M/cnpy.cpp:104-153).  Host only.
#pragma once

#include <cstddef>
#include <string>
#include <vector>

namespace msd {
namespace npy {

struct Array {
    std::vector<size_t> shape;
    std::vector<float> data;
    size_t num_vals() const { return data.size(); }
};

// Throws std::runtime_error("npy_load: Unable to open file <path>") when the file cannot be
// opened (the reference's message, M/util.cpp:111), and a "parse_npy_header: ..." /
// "npy_load: ..." error for a malformed header, a dtype other than '<f4', Fortran order or
// a payload shorter than the shape promises.
Array load(const std::string &path);

// Writes version 1.0 with a 64-byte-aligned header, as numpy.save does.
void save(const std::string &path, const std::vector<size_t> &shape, const float *data);

}  // namespace npy
}  // namespace msd
