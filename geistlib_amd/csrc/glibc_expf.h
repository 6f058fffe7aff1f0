/*
 * glibc_expf.h -- expf with the exact results of glibc 2.35's expf on an FMA-capable x86-64.
 *
 * The reference sampler calls libm expf (src/engine/sampler.c:80). Token ids only agree
 * with it bit for bit if each probability does, so the device evaluates the same algorithm
 * glibc uses (sysdeps/ieee754/flt-32/e_expf.c, from ARM's optimized-routines, MIT licence):
 *   x * 32/ln2 = k + r,  r in [-1/2, 1/2];  exp(x) = 2^(k/32) * P(r),
 * with 2^(i/32) from a 32-entry table of correctly rounded doubles, a cubic P, every step in
 * binary64 and one final rounding to binary32. The x86-64 build selected on FMA hardware
 * contracts each multiply-add, which is what the fma() calls below restate; with them the
 * function equals libm expf for every one of the 1 120 927 745 floats in [-104, 0] (checked
 * exhaustively on the host, see tests/test_expf_exact.py). Without contraction a single input
 * in that range rounds differently.
 *
 * Compiles as host C++ and as HIP device code.
 */
#ifndef GEIST_GLIBC_EXPF_H
#define GEIST_GLIBC_EXPF_H

#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define GEIST_HD __host__ __device__ __forceinline__
#else
#include <math.h>
#define GEIST_HD static inline
#endif

/* bits of 2^(i/32) minus (i << 47): adding (k << 47) then yields 2^(k/32) with the exponent
 * carried by k / 32. */
#define GEIST_EXPF_TABLE_INIT                                                                  \
    {                                                                                          \
        0x3ff0000000000000ULL, 0x3fefd9b0d3158574ULL, 0x3fefb5586cf9890fULL,                   \
        0x3fef9301d0125b51ULL, 0x3fef72b83c7d517bULL, 0x3fef54873168b9aaULL,                   \
        0x3fef387a6e756238ULL, 0x3fef1e9df51fdee1ULL, 0x3fef06fe0a31b715ULL,                   \
        0x3feef1a7373aa9cbULL, 0x3feedea64c123422ULL, 0x3feece086061892dULL,                   \
        0x3feebfdad5362a27ULL, 0x3feeb42b569d4f82ULL, 0x3feeab07dd485429ULL,                   \
        0x3feea47eb03a5585ULL, 0x3feea09e667f3bcdULL, 0x3fee9f75e8ec5f74ULL,                   \
        0x3feea11473eb0187ULL, 0x3feea589994cce13ULL, 0x3feeace5422aa0dbULL,                   \
        0x3feeb737b0cdc5e5ULL, 0x3feec49182a3f090ULL, 0x3feed503b23e255dULL,                   \
        0x3feee89f995ad3adULL, 0x3feeff76f2fb5e47ULL, 0x3fef199bdd85529cULL,                   \
        0x3fef3720dcef9069ULL, 0x3fef5818dcfba487ULL, 0x3fef7c97337b9b5fULL,                   \
        0x3fefa4afa2a490daULL, 0x3fefd0765b6e4540ULL                                           \
    }

GEIST_HD double geist_u64_as_double(uint64_t u) {
    double d;
    memcpy(&d, &u, sizeof d);
    return d;
}
GEIST_HD uint64_t geist_double_as_u64(double d) {
    uint64_t u;
    memcpy(&u, &d, sizeof u);
    return u;
}
GEIST_HD uint32_t geist_float_as_u32(float f) {
    uint32_t u;
    memcpy(&u, &f, sizeof u);
    return u;
}

/* `tab` points at the 32 table words (LDS, constant or host memory). */
GEIST_HD float geist_expf_glibc(float x, const uint64_t *tab) {
    const uint32_t ix     = geist_float_as_u32(x);
    const uint32_t abstop = (ix >> 20) & 0x7ff;
    if (abstop >= 0x42b) { /* |x| >= 88 or NaN */
        if (ix == 0xff800000u)
            return 0.0f; /* -inf */
        if (abstop >= 0x7f8)
            return x + x; /* +inf, NaN */
        if (x > 0x1.62e42ep6f)
            return __builtin_inff(); /* overflow */
        if (x < -0x1.9fe368p6f)
            return 0.0f; /* below 2^-150 */
    }
    const double inv_ln2_n = 0x1.71547652b82fep+0 * 32.0;
    const double shift     = 0x1.8p+52;
    const double c0        = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0;
    const double c1        = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0;
    const double c2        = 0x1.62e42ff0c52d6p-1 / 32.0;

    const double   xd = (double) x;
    double         kd = __builtin_fma(inv_ln2_n, xd, shift);
    const uint64_t ki = geist_double_as_u64(kd);
    kd -= shift;
    const double r = __builtin_fma(inv_ln2_n, xd, -kd);
    uint64_t     t = tab[ki & 31];
    t += ki << 47;
    const double s  = geist_u64_as_double(t);
    const double z  = __builtin_fma(c0, r, c1);
    const double r2 = r * r;
    double       y  = __builtin_fma(c2, r, 1.0);
    y               = __builtin_fma(z, r2, y);
    y               = y * s;
    return (float) y;
}

/* The same function for arguments x <= 0 (and NaN), without branches or selects, so that the
 * compiler can interleave the evaluations of many elements: arguments below -104 are raised to
 * -104, where the polynomial's result already rounds to 0 as every smaller argument's does (the
 * underflow edge -103.972 is where the rounding of the same expression flips), and a NaN runs
 * through the arithmetic and comes out a NaN. Equal to geist_expf_glibc() on every such input
 * (checked exhaustively). A positive argument is outside the contract: the sampler's arguments
 * are (l - max) * inv_t with max taken over the same values. */
GEIST_HD float geist_expf_glibc_le0(float x, const uint64_t *tab) {
    const double inv_ln2_n = 0x1.71547652b82fep+0 * 32.0;
    const double shift     = 0x1.8p+52;
    const double c0        = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0;
    const double c1        = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0;
    const double c2        = 0x1.62e42ff0c52d6p-1 / 32.0;

    const float    xc = x < -104.0f ? -104.0f : x; /* a NaN compares false and stays */
    const double   xd = (double) xc;
    double         kd = __builtin_fma(inv_ln2_n, xd, shift);
    const uint64_t ki = geist_double_as_u64(kd);
    kd -= shift;
    const double   r  = __builtin_fma(inv_ln2_n, xd, -kd);
    /* ki << 47 only reaches the high word: add (low word of ki) << 15 there, in 32-bit
     * arithmetic (one shift-add on the device) */
    typedef uint32_t geist_u32x2 __attribute__((vector_size(8)));
    const uint32_t kl = (uint32_t) ki;
    geist_u32x2    w  = __builtin_bit_cast(geist_u32x2, tab[kl & 31]);
    w[1] += kl << 15;
    const double s = __builtin_bit_cast(double, w);
    const double   z  = __builtin_fma(c0, r, c1);
    const double   r2 = r * r;
    double         y  = __builtin_fma(c2, r, 1.0);
    y                 = __builtin_fma(z, r2, y);
    y                 = y * s;
    return (float) y;
}

/* Any argument: positive ones take the general function. */
GEIST_HD float geist_expf_glibc_nonpos(float x, const uint64_t *tab) {
    if (__builtin_expect(x > 0.0f, 0))
        return geist_expf_glibc(x, tab);
    return geist_expf_glibc_le0(x, tab);
}

#endif /* GEIST_GLIBC_EXPF_H */
