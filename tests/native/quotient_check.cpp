// Host build of geist_quotient_f32 (geistlib_amd/csrc/exact_quotient.h) compared with the
// division it stands for, (float) ((double) p / tot). Inputs: p a binary32 in (0, 1] (what expf
// of a non-positive argument gives, with every exponent down to the subnormals), tot a double
// of at least 1 (the row's sum). A share of the cases is built to be hard: tot is chosen so that
// p / tot falls within a rounding error of the middle between two binary32 values, where the
// choice of the neighbouring double decides the result. Prints the number of cases whose
// results differ in any bit, the number of cases, and how many took the division because the
// quotient lay beside a middle, and because it was tiny.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../geistlib_amd/csrc/exact_quotient.h"

static inline uint64_t next(uint64_t &s) {
    s ^= s << 13;
    s ^= s >> 7;
    s ^= s << 17;
    return s;
}

int main(int argc, char **argv) {
    const long n    = argc > 1 ? atol(argv[1]) : 10000000L;
    const int  part = argc > 2 ? atoi(argv[2]) : 16;
    long       bad = 0, beside = 0, tiny = 0;
#pragma omp parallel for reduction(+ : bad, beside, tiny) schedule(static)
    for (int t = 0; t < part; ++t) {
        uint64_t s = 88172645463325252ull + 0x9E3779B97F4A7C15ull * (uint64_t) (t + 1);
        for (long i = 0; i < n / part; ++i) {
            uint32_t pb = (uint32_t) next(s) & 0x007fffffu;
            int      e  = 127 - (int) (next(s) % 150); /* exponents 127 .. -22: subnormals too */
            if (e < 0)
                e = 0;
            pb |= (uint32_t) e << 23;
            float p;
            memcpy(&p, &pb, 4);
            if (i % 7 == 0)
                p = 1.0f; /* the row's largest element */
            double tot = 1.0 + (double) (next(s) >> 11) * 0x1p-53 * 3.0e5;
            if (i % 5 == 0)
                tot = 1.0 + (double) (next(s) >> 40); /* integers */
            if (i % 3 == 0 && p > 0x1p-100f) {
                /* a middle between two binary32 values below p, and the sum that puts p / tot there */
                uint32_t fb = (uint32_t) next(s) & 0x007fffffu;
                int      fe = (int) (pb >> 23) - 1 - (int) (next(s) % 18);
                if (fe < 2)
                    fe = 2;
                fb |= (uint32_t) fe << 23;
                float f;
                memcpy(&f, &fb, 4);
                const double mid = (double) f + ldexp(1.0, fe - 127 - 24);
                const double tt  = (double) p / mid;
                if (tt >= 1.0 && std::isfinite(tt))
                    tot = tt;
            }
            const double rtot = 1.0 / tot;
            const float  a = geist_quotient_f32(p, tot, rtot), b = (float) ((double) p / tot);
            {
                /* the same tests as in the header, to count the cases that took the division */
                const double pd = (double) p;
                double       q  = pd * rtot;
                q               = __builtin_fma(__builtin_fma(-q, tot, pd), rtot, q);
                uint64_t qb;
                memcpy(&qb, &q, 8);
                const uint32_t low = (uint32_t) qb & 0x1fffffffu;
                const int      ex  = (int) ((qb >> 52) & 0x7ff);
                if (ex < 1023 - 120 || ex == 0x7ff)
                    ++tiny;
                else if ((low - 0x0ffffffeu) <= 4u)
                    ++beside;
            }
            if (memcmp(&a, &b, 4) != 0)
                ++bad;
        }
    }
    printf("%ld %ld %ld %ld\n", bad, (n / part) * part, beside, tiny);
    return 0;
}
