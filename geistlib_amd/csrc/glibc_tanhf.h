/*
 * glibc_tanhf.h -- tanhf with the exact results of glibc 2.35's tanhf on x86-64.
 *
 * The reference applies its logit soft-cap with libm: tanhf(x / cap) * cap
 * (src/archs/transformer/forward/head.c:148-159, 279-288). A capped logit that differs in its
 * last bit moves a probability and can move a token, so the device evaluates the algorithm glibc
 * 2.35 uses: the fdlibm tanhf (sysdeps/ieee754/flt-32/s_tanhf.c) over the fdlibm expm1f
 * (s_expm1f.c), all in binary32 with every operation rounded on its own. The x86-64 baseline
 * build has no fused multiply-add, so nothing here may be contracted: each step goes through
 * gs_f* helpers that are rounding intrinsics on the device and plain operators on the host
 * (compile the host side with -ffp-contract=off).
 *
 * The restatement equals libm tanhf for every binary32 input (checked exhaustively on the host,
 * tests/test_tanhf_exact.py).
 *
 * Compiles as host C++ and as HIP device code.
 */
#ifndef GEIST_GLIBC_TANHF_H
#define GEIST_GLIBC_TANHF_H

#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define GEIST_TH_HD __host__ __device__ __forceinline__
#else
#define GEIST_TH_HD static inline
#endif

#if defined(__HIP_DEVICE_COMPILE__)
#define gs_fadd(a, b) __fadd_rn((a), (b))
#define gs_fsub(a, b) __fsub_rn((a), (b))
#define gs_fmul(a, b) __fmul_rn((a), (b))
#define gs_fdiv(a, b) __fdiv_rn((a), (b))
#else
#define gs_fadd(a, b) ((float) ((a) + (b)))
#define gs_fsub(a, b) ((float) ((a) - (b)))
#define gs_fmul(a, b) ((float) ((a) * (b)))
#define gs_fdiv(a, b) ((float) ((a) / (b)))
#endif

GEIST_TH_HD uint32_t geist_th_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, sizeof u);
    return u;
}
GEIST_TH_HD float geist_th_float(uint32_t u) {
    float f;
    memcpy(&f, &u, sizeof f);
    return f;
}

/* expm1f of fdlibm for the arguments tanhf feeds it: finite, |x| < 44. */
GEIST_TH_HD float geist_expm1f_fdlibm(float x) {
    const float one = 1.0f, ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f,
                invln2 = 1.4426950216e+00f, Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f,
                Q3 = -7.9365076090e-05f, Q4 = 4.0082177293e-06f, Q5 = -2.0109921195e-07f;
    uint32_t       hx  = geist_th_bits(x);
    const uint32_t xsb = hx & 0x80000000u;
    hx &= 0x7fffffffu;
    float   hi, lo, c = 0.0f, t, e, hxs, hfx, r1, y;
    int32_t k;
    if (hx >= 0x4195b844u) { /* |x| >= 27 ln2 */
        if (hx >= 0x42b17218u) {
            if (hx > 0x7f800000u)
                return gs_fadd(x, x);
            if (hx == 0x7f800000u)
                return xsb == 0 ? x : -1.0f;
            if (x > 8.8721679688e+01f)
                return __builtin_inff();
        }
        if (xsb != 0)
            return gs_fsub(1.0e-30f, one); /* -1 */
    }
    if (hx > 0x3eb17218u) { /* |x| > 0.5 ln2 */
        if (hx < 0x3F851592u) { /* |x| < 1.5 ln2 */
            if (xsb == 0) {
                hi = gs_fsub(x, ln2_hi);
                lo = ln2_lo;
                k  = 1;
            } else {
                hi = gs_fadd(x, ln2_hi);
                lo = -ln2_lo;
                k  = -1;
            }
        } else {
            k  = (int32_t) gs_fadd(gs_fmul(invln2, x), xsb == 0 ? 0.5f : -0.5f);
            t  = (float) k;
            hi = gs_fsub(x, gs_fmul(t, ln2_hi)); /* t * ln2_hi is exact here */
            lo = gs_fmul(t, ln2_lo);
        }
        x = gs_fsub(hi, lo);
        c = gs_fsub(gs_fsub(hi, x), lo);
    } else if (hx < 0x33000000u) { /* |x| < 2^-25 */
        t = gs_fadd(1.0e+30f, x);
        return gs_fsub(x, gs_fsub(t, gs_fadd(1.0e+30f, x)));
    } else {
        k = 0;
    }
    hfx = gs_fmul(0.5f, x);
    hxs = gs_fmul(x, hfx);
    r1  = gs_fadd(Q4, gs_fmul(hxs, Q5));
    r1  = gs_fadd(Q3, gs_fmul(hxs, r1));
    r1  = gs_fadd(Q2, gs_fmul(hxs, r1));
    r1  = gs_fadd(Q1, gs_fmul(hxs, r1));
    r1  = gs_fadd(one, gs_fmul(hxs, r1));
    t   = gs_fsub(3.0f, gs_fmul(r1, hfx));
    e   = gs_fmul(hxs, gs_fdiv(gs_fsub(r1, t), gs_fsub(6.0f, gs_fmul(x, t))));
    if (k == 0)
        return gs_fsub(x, gs_fsub(gs_fmul(x, e), hxs));
    e = gs_fsub(gs_fmul(x, gs_fsub(e, c)), c);
    e = gs_fsub(e, hxs);
    if (k == -1)
        return gs_fsub(gs_fmul(0.5f, gs_fsub(x, e)), 0.5f);
    if (k == 1) {
        if (x < -0.25f)
            return gs_fmul(-2.0f, gs_fsub(e, gs_fadd(x, 0.5f)));
        return gs_fadd(one, gs_fmul(2.0f, gs_fsub(x, e)));
    }
    if (k <= -2 || k > 56) {
        y = gs_fsub(one, gs_fsub(e, x));
        y = geist_th_float(geist_th_bits(y) + ((uint32_t) k << 23));
        return gs_fsub(y, one);
    }
    if (k < 23) {
        t = geist_th_float(0x3f800000u - (0x1000000u >> k)); /* 1 - 2^-k */
        y = gs_fsub(t, gs_fsub(e, x));
        y = geist_th_float(geist_th_bits(y) + ((uint32_t) k << 23));
    } else {
        t = geist_th_float((uint32_t) (0x7f - k) << 23); /* 2^-k */
        y = gs_fsub(x, gs_fadd(e, t));
        y = gs_fadd(y, one);
        y = geist_th_float(geist_th_bits(y) + ((uint32_t) k << 23));
    }
    return y;
}

GEIST_TH_HD float geist_tanhf_glibc(float x) {
    const float    one = 1.0f, two = 2.0f;
    const uint32_t jx = geist_th_bits(x), ix = jx & 0x7fffffffu;
    float          t, z;
    if (!(ix < 0x7f800000u)) { /* inf or NaN */
        if ((int32_t) jx >= 0)
            return gs_fadd(gs_fdiv(one, x), one);
        return gs_fsub(gs_fdiv(one, x), one);
    }
    if (ix < 0x41b00000u) { /* |x| < 22 */
        if (ix == 0)
            return x;
        if (ix < 0x24000000u) /* |x| < 2^-55 */
            return gs_fmul(x, gs_fadd(one, x));
        const float ax = geist_th_float(ix);
        if (ix >= 0x3f800000u) { /* |x| >= 1 */
            t = geist_expm1f_fdlibm(gs_fmul(two, ax));
            z = gs_fsub(one, gs_fdiv(two, gs_fadd(t, two)));
        } else {
            t = geist_expm1f_fdlibm(gs_fmul(-two, ax));
            z = gs_fdiv(-t, gs_fadd(t, two));
        }
    } else {
        z = gs_fsub(one, 1.0e-30f);
    }
    return (int32_t) jx >= 0 ? z : -z;
}

#endif /* GEIST_GLIBC_TANHF_H */
