// msd_compare: compares two .npy files (little-endian float32, C order) the way the
// reference's util::testBuffer compares a device buffer with a golden file
// (M/util.cpp:167-201): elements that differ at all are counted, the largest absolute
// difference and its index are reported in the same one-line format.  Host only; used
// to check outputs dumped by a deployment against fixtures without a GPU at hand.
//
//   msd_compare RESULT.npy GOLDEN.npy [--rel TOL] [--abs TOL] [--show N]
//
// Exit status: 0 when every element satisfies |r - g| <= max(abs, rel * max(1, |g|))
// (defaults: rel 1e-5, abs 0, the float32 criterion of the parity tests), 1 when some
// element does not, 2 for usage / file / size errors.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <string>
#include <vector>

#include "npy.h"

int main(int argc, char **argv) {
    double rel = 1e-5, abs_tol = 0.0;
    long show = 10;  // the reference logs the first 10 mismatches
    std::vector<std::string> files;
    for (int i = 1; i < argc; i++) {
        const std::string a = argv[i];
        if ((a == "--rel" || a == "--abs" || a == "--show") && i + 1 < argc) {
            const double v = atof(argv[++i]);
            if (a == "--rel") rel = v;
            else if (a == "--abs") abs_tol = v;
            else show = (long)v;
        } else if (!a.empty() && a[0] == '-') {
            fprintf(stderr, "unknown option %s\n", a.c_str());
            return 2;
        } else {
            files.push_back(a);
        }
    }
    if (files.size() != 2) {
        fprintf(stderr, "usage: msd_compare RESULT.npy GOLDEN.npy [--rel TOL] [--abs TOL] [--show N]\n");
        return 2;
    }
    msd::npy::Array result, test;
    try {
        result = msd::npy::load(files[0]);
        test = msd::npy::load(files[1]);
    } catch (const std::exception &e) {
        fprintf(stderr, "%s\n", e.what());
        return 2;
    }
    if (result.num_vals() != test.num_vals()) {
        fprintf(stderr, "%s: bufferSize(%zu) != test.num_vals(%zu)\n", files[1].c_str(), result.num_vals(),
                test.num_vals());
        return 2;
    }
    float max_diff = 0.0f;
    size_t max_id = 0, num_wrong = 0, out_of_tolerance = 0;
    std::vector<size_t> first;
    for (size_t i = 0; i < test.num_vals(); i++) {
        const float r = result.data[i], g = test.data[i];
        if (r != g) {
            num_wrong++;
            if ((long)first.size() < show) first.push_back(i);
            const float diff = std::fabs(r - g);
            if (diff > max_diff || std::isnan(diff)) {
                max_diff = diff;
                max_id = i;
            }
            const double bound = std::fmax(abs_tol, rel * std::fmax(1.0, std::fabs((double)g)));
            if (!((double)diff <= bound)) out_of_tolerance++;
        }
    }
    if (test.num_vals() != 0)
        printf("%s max diff: %.20f / num : %zu / result[%zu]: %f/ test[%zu]: %f\n", files[1].c_str(), max_diff,
               num_wrong, max_id, result.data[max_id], max_id, test.data[max_id]);
    for (size_t i : first) printf("result[%zu]: %f != test[%zu]: %f\n", i, result.data[i], i, test.data[i]);
    printf("%zu of %zu elements outside |r-g| <= max(%g, %g*max(1,|g|))\n", out_of_tolerance, test.num_vals(),
           abs_tol, rel);
    return out_of_tolerance == 0 ? 0 : 1;
}
