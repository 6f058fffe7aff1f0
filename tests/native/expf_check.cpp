// Host build of the device expf (geistlib_amd/csrc/glibc_expf.h) compared with libm expf.
// Prints the number of floats in the given bit range whose results differ in any bit.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../geistlib_amd/csrc/glibc_expf.h"

static const uint64_t TAB[32] = GEIST_EXPF_TABLE_INIT;

int main(int argc, char **argv) {
    const uint32_t lo = argc > 1 ? (uint32_t) strtoul(argv[1], nullptr, 0) : 0x80000000u;
    const uint32_t hi = argc > 2 ? (uint32_t) strtoul(argv[2], nullptr, 0) : 0xc2d00000u; /* -104 */
    long           bad = 0, total = 0;
#pragma omp parallel for reduction(+ : bad, total) schedule(static)
    for (int64_t b = lo; b <= (int64_t) hi; ++b) {
        const uint32_t u = (uint32_t) b;
        float          x;
        memcpy(&x, &u, 4);
        const float want = expf(x), got = geist_expf_glibc(x, TAB),
                    got2 = geist_expf_glibc_nonpos(x, TAB),
                    /* the branch-free variant, defined for x <= 0 and NaN */
                    got3 = x > 0.0f ? want : geist_expf_glibc_le0(x, TAB);
        uint32_t    uw, ug, ug2, ug3;
        memcpy(&uw, &want, 4);
        memcpy(&ug, &got, 4);
        memcpy(&ug2, &got2, 4);
        memcpy(&ug3, &got3, 4);
        const bool both_nan  = want != want && got != got;
        const bool both_nan2 = want != want && got2 != got2;
        const bool both_nan3 = want != want && got3 != got3;
        ++total;
        if ((uw != ug && !both_nan) || (uw != ug2 && !both_nan2) || (uw != ug3 && !both_nan3))
            ++bad;
    }
    printf("%ld %ld\n", bad, total);
    return 0;
}
