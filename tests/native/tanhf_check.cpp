// Host build of the device tanhf (geistlib_amd/csrc/glibc_tanhf.h) compared with libm tanhf.
// Prints the number of floats in the given bit range whose results differ in any bit, the number
// of floats tried, and the first differing input.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../geistlib_amd/csrc/glibc_tanhf.h"

// "mono" as third argument: counts instead the floats x in the range whose successor has a
// smaller tanhf (the function would then not be monotone); same three numbers.
static int monotone(uint32_t lo, uint32_t hi) {
    long    bad = 0, total = 0;
    int64_t first = -1;
#pragma omp parallel for reduction(+ : bad, total) schedule(static)
    for (int64_t b = lo; b < (int64_t) hi; ++b) {
        const uint32_t u0 = (uint32_t) b, u1 = u0 + 1u;
        float          x0, x1;
        memcpy(&x0, &u0, 4);
        memcpy(&x1, &u1, 4);
        ++total;
        if (geist_tanhf_glibc(x1) < geist_tanhf_glibc(x0)) {
            ++bad;
#pragma omp critical
            if (first < 0 || b < first)
                first = b;
        }
    }
    printf("%ld %ld %lld\n", bad, total, (long long) first);
    return 0;
}

int main(int argc, char **argv) {
    const uint32_t lo = argc > 1 ? (uint32_t) strtoul(argv[1], nullptr, 0) : 0u;
    const uint32_t hi = argc > 2 ? (uint32_t) strtoul(argv[2], nullptr, 0) : 0x7f800000u;
    if (argc > 3 && strcmp(argv[3], "mono") == 0)
        return monotone(lo, hi);
    long           bad = 0, total = 0;
    int64_t        first = -1;
#pragma omp parallel for reduction(+ : bad, total) schedule(static)
    for (int64_t b = lo; b <= (int64_t) hi; ++b) {
        const uint32_t u = (uint32_t) b;
        float          x;
        memcpy(&x, &u, 4);
        const float want = tanhf(x), got = geist_tanhf_glibc(x);
        uint32_t    uw, ug;
        memcpy(&uw, &want, 4);
        memcpy(&ug, &got, 4);
        const bool both_nan = want != want && got != got;
        ++total;
        if (uw != ug && !both_nan) {
            ++bad;
#pragma omp critical
            if (first < 0 || b < first)
                first = b;
        }
    }
    printf("%ld %ld %lld\n", bad, total, (long long) first);
    return 0;
}
