#include "npy.h"

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <stdexcept>

namespace msd {
namespace npy {
namespace {

struct File {
    FILE *fp;
    explicit File(FILE *f) : fp(f) {}
    ~File() {
        if (fp) fclose(fp);
    }
};

// value text following "'key':" in the header dictionary
std::string dict_value(const std::string &header, const char *key) {
    const std::string quoted = std::string("'") + key + "'";
    size_t at = header.find(quoted);
    if (at == std::string::npos)
        throw std::runtime_error(std::string("parse_npy_header: failed to find header keyword: '") +
                                 key + "'");
    at = header.find(':', at + quoted.size());
    if (at == std::string::npos) throw std::runtime_error("parse_npy_header: malformed dictionary");
    at++;
    while (at < header.size() && header[at] == ' ') at++;
    return header.substr(at);
}

}  // namespace

Array load(const std::string &path) {
    File f(fopen(path.c_str(), "rb"));
    if (!f.fp) throw std::runtime_error("npy_load: Unable to open file " + path);
    unsigned char pre[10];
    if (fread(pre, 1, 10, f.fp) != 10) throw std::runtime_error("parse_npy_header: failed fread");
    if (memcmp(pre, "\x93NUMPY", 6) != 0) throw std::runtime_error("parse_npy_header: not an NPY file");
    const int major = pre[6];
    size_t header_len = 0;
    if (major == 1) {
        header_len = (size_t)pre[8] | ((size_t)pre[9] << 8);
    } else if (major == 2 || major == 3) {
        unsigned char more[2];
        if (fread(more, 1, 2, f.fp) != 2) throw std::runtime_error("parse_npy_header: failed fread");
        header_len = (size_t)pre[8] | ((size_t)pre[9] << 8) | ((size_t)more[0] << 16) |
                     ((size_t)more[1] << 24);
    } else {
        throw std::runtime_error("parse_npy_header: unsupported NPY version");
    }
    if (header_len == 0 || header_len > (1u << 20))
        throw std::runtime_error("parse_npy_header: bad header length");
    std::string header(header_len, '\0');
    if (fread(&header[0], 1, header_len, f.fp) != header_len)
        throw std::runtime_error("parse_npy_header: failed fread");

    const std::string descr = dict_value(header, "descr");
    if (descr.size() < 5 || (descr[0] != '\'' && descr[0] != '"'))
        throw std::runtime_error("parse_npy_header: malformed descr");
    const std::string type = descr.substr(1, 3);
    if (type != "<f4")
        throw std::runtime_error("npy_load: expected little-endian float32 ('<f4') data, found '" +
                                 type + "' in " + path);
    if (dict_value(header, "fortran_order").compare(0, 4, "True") == 0)
        throw std::runtime_error("npy_load: Fortran-ordered arrays are not supported: " + path);

    const std::string shape_text = dict_value(header, "shape");
    const size_t open = shape_text.find('('), close = shape_text.find(')');
    if (open != 0 || close == std::string::npos)
        throw std::runtime_error("parse_npy_header: failed to find header keyword: '(' or ')'");
    // what is left of the file bounds the element count: a header that claims more is refused
    // before anything is allocated, and the running product cannot overflow below that bound
    const long data_start = ftell(f.fp);
    if (data_start < 0 || fseek(f.fp, 0, SEEK_END) != 0) throw std::runtime_error("npy_load: cannot seek in " + path);
    const long file_end = ftell(f.fp);
    if (file_end < data_start || fseek(f.fp, data_start, SEEK_SET) != 0)
        throw std::runtime_error("npy_load: cannot seek in " + path);
    const size_t max_vals = (size_t)(file_end - data_start) / sizeof(float);
    Array out;
    size_t total = 1;
    size_t i = open + 1;
    while (i < close) {
        if (shape_text[i] >= '0' && shape_text[i] <= '9') {
            size_t v = 0;
            while (i < close && shape_text[i] >= '0' && shape_text[i] <= '9') {
                if (v > max_vals) throw std::runtime_error("nread != num_bytes");  // longer than the file
                v = v * 10 + (size_t)(shape_text[i++] - '0');
            }
            out.shape.push_back(v);
            if (v != 0 && total > max_vals / v) throw std::runtime_error("nread != num_bytes");
            total *= v;
        } else {
            i++;
        }
    }
    out.data.resize(total);
    const size_t nread = total ? fread(out.data.data(), sizeof(float), total, f.fp) : 0;
    if (nread != total) throw std::runtime_error("nread != num_bytes");  // M/util.cpp:140
    return out;
}

void save(const std::string &path, const std::vector<size_t> &shape, const float *data) {
    std::string dict = "{'descr': '<f4', 'fortran_order': False, 'shape': (";
    size_t total = 1;
    for (size_t d = 0; d < shape.size(); d++) {
        dict += std::to_string(shape[d]);
        if (shape.size() == 1 || d + 1 < shape.size()) dict += ",";
        if (d + 1 < shape.size()) dict += " ";
        total *= shape[d];
    }
    dict += "), }";
    while ((10 + dict.size() + 1) % 64 != 0) dict += ' ';
    dict += '\n';
    File f(fopen(path.c_str(), "wb"));
    if (!f.fp) throw std::runtime_error("npy_save: Unable to open file " + path);
    const unsigned char pre[10] = {0x93, 'N', 'U', 'M', 'P', 'Y', 1, 0,
                                   (unsigned char)(dict.size() & 0xFF),
                                   (unsigned char)(dict.size() >> 8)};
    if (fwrite(pre, 1, 10, f.fp) != 10 || fwrite(dict.data(), 1, dict.size(), f.fp) != dict.size() ||
        (total && fwrite(data, sizeof(float), total, f.fp) != total))
        throw std::runtime_error("npy_save: short write to " + path);
}

}  // namespace npy
}  // namespace msd
