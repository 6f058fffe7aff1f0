/*
 * exact_quotient.h -- (float) ((double) p / tot) without the division.
 *
 * The reference normalises every probability as (float) ((double) p / sum)
 * (src/engine/sampler.c:246-253). With r = 1 / tot correctly rounded, q0 = p r and the exact
 * remainder e = p - q0 tot (one fused multiply-add: the product is exact there), q = q0 + e r
 * is the correctly rounded quotient or its neighbour. Both round to the same binary32 unless
 * they lie next to the middle between two binary32 values, or the result is too small for a
 * normal binary32, infinite or not a number: in those cases the division itself is taken.
 * Checked against the division on the host (tests/test_quotient_exact.py).
 *
 * Compiles as host C++ and as HIP device code.
 */
#ifndef GEIST_EXACT_QUOTIENT_H
#define GEIST_EXACT_QUOTIENT_H

#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define GEIST_QHD __host__ __device__ __forceinline__
#else
#include <math.h>
#define GEIST_QHD static inline
#endif

/* `rtot` is 1.0 / tot, computed once per row by the caller. */
GEIST_QHD float geist_quotient_f32(float p, double tot, double rtot) {
    const double pd = (double) p;
    double       q  = pd * rtot;
    const double e  = __builtin_fma(-q, tot, pd);
    q               = __builtin_fma(e, rtot, q);
    uint64_t b;
    memcpy(&b, &q, sizeof b);
    const uint32_t low = (uint32_t) b & 0x1fffffffu; /* the 29 bits that a binary32 drops */
    const int      ex  = (int) ((b >> 52) & 0x7ff);
    /* within two units of the middle (bit 28 set, the rest clear), or a result below 2^-120,
     * infinite or not a number */
    if ((low - 0x0ffffffeu) <= 4u || ex < 1023 - 120 || ex == 0x7ff)
        return (float) (pd / tot);
    return (float) q;
}

#endif
