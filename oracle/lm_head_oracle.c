/*
 * lm_head_oracle.c -- see lm_head_oracle.h. Test infrastructure only.
 */
#include "lm_head_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* src/formats/gguf/common.c:29-62 */
float oracle_f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t) (h >> 15) << 31;
    const uint32_t e    = (h >> 10) & 0x1fu;
    uint32_t       m    = h & 0x3ffu;
    uint32_t       bits;
    if (e == 0x1fu) {
        bits = sign | 0x7f800000u | (m << 13);
    } else if (e != 0) {
        bits = sign | ((e + 112u) << 23) | (m << 13);
    } else if (m == 0) {
        bits = sign;
    } else { /* subnormal: value m * 2^-24, normalised */
        uint32_t e32 = 113u;
        while (!(m & 0x400u)) {
            m <<= 1;
            e32--;
        }
        bits = sign | (e32 << 23) | ((m & 0x3ffu) << 13);
    }
    float f;
    memcpy(&f, &bits, sizeof f);
    return f;
}

uint16_t oracle_f32_to_f16(float v) {
    uint32_t b;
    memcpy(&b, &v, sizeof b);
    const uint16_t sign = (uint16_t) ((b >> 16) & 0x8000u);
    const uint32_t a    = b & 0x7fffffffu;
    if (a >= 0x7f800000u) /* inf, NaN (quiet) */
        return (uint16_t) (sign | 0x7c00u | (a > 0x7f800000u ? 0x200u | ((a >> 13) & 0x3ffu) : 0u));
    if (a >= 0x477ff000u) /* rounds to or beyond 65520 */
        return (uint16_t) (sign | 0x7c00u);
    if (a < 0x33000001u) /* at most half of the smallest subnormal */
        return sign;
    int      e = (int) (a >> 23) - 127;
    uint32_t m = (a & 0x7fffffu) | 0x800000u;
    int      shift;
    uint32_t base;
    if (e < -14) { /* subnormal result: value = m * 2^(e-23), unit 2^-24 */
        shift = -1 - e; /* 13 + (-14 - e) */
        base  = 0;
    } else {
        shift = 13;
        base  = (uint32_t) (e + 15) << 10;
        m &= 0x7fffffu;
    }
    const uint32_t q    = m >> shift;
    const uint32_t rem  = m & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    uint32_t       r    = base + q;
    if (rem > half || (rem == half && (q & 1u)))
        r++; /* carries into the exponent as it should */
    return (uint16_t) (sign | r);
}

/* src/backends/cpu_x86/kernel_f16_gemv.c:34-64 */
void oracle_f16_gemv_m1(size_t n_out, size_t n_in, const float *x, const uint16_t *w_f16, float *y) {
    for (size_t r = 0; r < n_out; r++) {
        const uint16_t *wr = w_f16 + r * n_in;
        float           chain[16];
        for (int j = 0; j < 16; j++)
            chain[j] = 0.0f;
        size_t k = 0;
        for (; k + 16 <= n_in; k += 16)
            for (int j = 0; j < 16; j++)
                chain[j] = fmaf(oracle_f16_to_f32(wr[k + j]), x[k + j], chain[j]);
        for (; k + 8 <= n_in; k += 8)
            for (int j = 0; j < 8; j++)
                chain[j] = fmaf(oracle_f16_to_f32(wr[k + j]), x[k + j], chain[j]);
        float v[8], q[4];
        for (int i = 0; i < 8; i++)
            v[i] = chain[i] + chain[i + 8];
        for (int i = 0; i < 4; i++)
            q[i] = v[i] + v[i + 4];
        float s = (q[0] + q[1]) + (q[2] + q[3]);
        for (; k < n_in; k++)
            s += oracle_f16_to_f32(wr[k]) * x[k];
        y[r] = s;
    }
}

/* src/backends/cpu_x86/kernel_f16_gemv.c:66-93 */
void oracle_f16_to_q8w(size_t n_out, size_t n_in, const uint16_t *w_f16, int8_t *wq, float *scales) {
    for (size_t r = 0; r < n_out; r++) {
        const uint16_t *wr   = w_f16 + r * n_in;
        float           amax = 0.0f;
        for (size_t k = 0; k < n_in; k++) {
            const float a = fabsf(oracle_f16_to_f32(wr[k]));
            if (a > amax)
                amax = a;
        }
        scales[r]      = amax / 127.0f;
        const float id = amax > 0.0f ? 127.0f / amax : 0.0f;
        for (size_t k = 0; k < n_in; k++) {
            long q = lrintf(oracle_f16_to_f32(wr[k]) * id);
            if (q > 127)
                q = 127;
            if (q < -127)
                q = -127;
            wq[r * n_in + k] = (int8_t) q;
        }
    }
}

/* src/backends/cpu_x86/kernel_f16_gemv.c:95-127 */
void oracle_q8w_gemv_m1(size_t n_out, size_t n_in, const float *x, const int8_t *wq,
                        const float *scales, float *y) {
    for (size_t r = 0; r < n_out; r++) {
        const int8_t *qr = wq + r * n_in;
        float         chain[16];
        for (int j = 0; j < 16; j++)
            chain[j] = 0.0f;
        size_t k = 0;
        for (; k + 16 <= n_in; k += 16)
            for (int j = 0; j < 16; j++)
                chain[j] = fmaf((float) qr[k + j], x[k + j], chain[j]);
        for (; k + 8 <= n_in; k += 8)
            for (int j = 0; j < 8; j++)
                chain[j] = fmaf((float) qr[k + j], x[k + j], chain[j]);
        float v[8], q[4];
        for (int i = 0; i < 8; i++)
            v[i] = chain[i] + chain[i + 8];
        for (int i = 0; i < 4; i++)
            q[i] = v[i] + v[i + 4];
        float s = (q[0] + q[1]) + (q[2] + q[3]);
        for (; k < n_in; k++)
            s += (float) qr[k] * x[k];
        y[r] = s * scales[r];
    }
}

/* src/backends/cpu_scalar/elementwise.c:266-278 */
void oracle_rmsnorm_rows(size_t n_rows, size_t n, const float *x, const float *w, float eps,
                         float *y) {
    for (size_t r = 0; r < n_rows; r++) {
        const float *xr    = x + r * n;
        double       sumsq = 0.0;
        for (size_t i = 0; i < n; i++)
            sumsq += (double) xr[i] * (double) xr[i];
        const float inv = (float) (1.0 / sqrt(sumsq / (double) n + (double) eps));
        for (size_t i = 0; i < n; i++)
            y[r * n + i] = xr[i] * inv * w[i];
    }
}


void oracle_f16_linear_f64(size_t m, size_t n_out, size_t n_in, const float *x,
                           const uint16_t *w_f16, float *y) {
    /* weight_resolve.c:221-238 with dequant_one_row_for's F16 case (:62-68) */
#pragma omp parallel for schedule(static)
    for (size_t j = 0; j < n_out; j++) {
        const uint16_t *wr = w_f16 + j * n_in;
        for (size_t i = 0; i < m; i++) {
            double acc = 0.0;
            for (size_t k = 0; k < n_in; k++)
                acc += (double) x[i * n_in + k] * (double) oracle_f16_to_f32(wr[k]);
            y[i * n_out + j] = (float) acc;
        }
    }
}

void oracle_dequant_q6_K_row(const void *blocks, float *out, size_t n_elems) {
    /* q6_K.c:13-45; the block layout of src/quant/quant_blocks.h:67-73 by offsets */
    const uint8_t *p = (const uint8_t *) blocks;
    for (size_t b = 0; b < n_elems / 256; b++, p += 210) {
        const uint8_t *ql = p, *qh = p + 128;
        const int8_t  *sc = (const int8_t *) (p + 192);
        const float    d  = oracle_f16_to_f32((uint16_t) (p[208] | (p[209] << 8)));
        float         *y  = out + b * 256;
        for (int h = 0; h < 2; h++)
            for (int j = 0; j < 4; j++)
                for (int l = 0; l < 32; l++) {
                    const uint8_t lo = ql[64 * h + 32 * (j & 1) + l];
                    const int     q  = (int) (((j >> 1) ? lo >> 4 : lo & 0xF) |
                                             (((qh[32 * h + l] >> (2 * j)) & 3) << 4)) - 32;
                    y[128 * h + 32 * j + l] = d * (float) sc[8 * h + 2 * j + l / 16] * (float) (int8_t) q;
                }
    }
}

void oracle_q6k_linear_f64(size_t m, size_t n_out, size_t n_in, const float *x,
                           const void *w_q6k, float *y) {
    /* weight_resolve.c:186-241 */
    const size_t row_bytes = n_in / 256 * 210;
#pragma omp parallel
    {
        float *row = (float *) malloc(n_in * sizeof(float));
#pragma omp for schedule(static)
        for (size_t j = 0; j < n_out; j++) {
            if (!row)
                continue;
            oracle_dequant_q6_K_row((const uint8_t *) w_q6k + j * row_bytes, row, n_in);
            for (size_t i = 0; i < m; i++) {
                double acc = 0.0;
                for (size_t k = 0; k < n_in; k++)
                    acc += (double) x[i * n_in + k] * (double) row[k];
                y[i * n_out + j] = (float) acc;
            }
        }
        free(row);
    }
}

/* ---- the x86 backend's decode kernel over a Q6_K table ---------------------------------------
 * src/backends/cpu_x86/kernel_q6k_gemv.c (q6k_gemv_m1, reached from cpu_x86_linear_q6k_m1,
 * linear_q6k.c:187-208, whenever the raw table is at hand): the activation row is quantised to
 * int8 per super-block of 256, the products are integers, and each super-block contributes one
 * binary32 multiply-add per lane of an eight-lane accumulator. Restated in scalar C: the AVX2
 * lanes become loops, every rounding stays where the vector code has it. */
void oracle_q8k_quantize(size_t n_super, const float *x, float *d_out, int8_t *qs_out,
                         int16_t *bsums_out) {
    /* kernel_q6k_gemv.c:43-67: d = amax / 127, qs = lrintf(x * (127 / amax)), sums per 16 */
    for (size_t s = 0; s < n_super; s++) {
        const float *xs   = x + s * 256;
        float        amax = 0.0f;
        for (int k = 0; k < 256; k++) {
            const float ax = fabsf(xs[k]);
            if (ax > amax)
                amax = ax;
        }
        const float id = amax > 0.0f ? 127.0f / amax : 0.0f;
        d_out[s]       = amax / 127.0f;
        for (int g = 0; g < 16; g++) {
            int sum = 0;
            for (int i = 0; i < 16; i++) {
                const int v = (int) lrintf(xs[g * 16 + i] * id);
                qs_out[s * 256 + g * 16 + i] = (int8_t) v;
                sum += v;
            }
            bsums_out[s * 16 + g] = (int16_t) sum;
        }
    }
}

/* One row's dot product, kernel_q6k_gemv.c:90-157. Lane u of the eight-lane integer sum takes,
 * from each of the super-block's eight runs of 32 elements, the four elements 4u .. 4u + 3 of
 * the run times the scale of their group of sixteen (run v, elements below 16: scale 2v, else
 * 2v + 1); the uniform offset of 32 leaves through the activations' sums per sixteen, which the
 * vector code pairs by SCALE index: lane u loses 32 (bsums[2u] scale[2u] + bsums[2u+1]
 * scale[2u+1]). Each lane's integer is converted to binary32 and joins the lane's accumulator by
 * one fused multiply-add with d = d_act * d_weight; the lanes are added as hsum_ps_avx adds them:
 * ((a0 + a4) + (a1 + a5)) + ((a2 + a6) + (a3 + a7)). */
static float oracle_dot_q6k_q8k(size_t n_super, const uint8_t *row, const float *d_act,
                                const int8_t *qs, const int16_t *bsums) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (size_t i = 0; i < n_super; i++, row += 210) {
        const uint8_t *ql = row, *qh = row + 128;
        const int8_t  *sc = (const int8_t *) (row + 192);
        const float    d  = d_act[i] * oracle_f16_to_f32((uint16_t) (row[208] | (row[209] << 8)));
        const int8_t  *q8 = qs + i * 256;
        int32_t        lane[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int v = 0; v < 8; v++) { /* run v: elements 32 v .. 32 v + 31 */
            const int h = v >> 2, j = v & 3;
            for (int b = 0; b < 32; b++) {
                const uint8_t lo = ql[64 * h + 32 * (j & 1) + b];
                const int     q  = ((j >> 1) ? lo >> 4 : lo & 0xF) | (((qh[32 * h + b] >> (2 * j)) & 3) << 4);
                lane[b >> 2] += (int32_t) sc[2 * v + (b >> 4)] * (q * (int32_t) q8[32 * v + b]);
            }
        }
        for (int u = 0; u < 8; u++) {
            lane[u] -= ((int32_t) bsums[i * 16 + 2 * u] * sc[2 * u] +
                        (int32_t) bsums[i * 16 + 2 * u + 1] * sc[2 * u + 1]) * 32;
            acc[u] = fmaf(d, (float) lane[u], acc[u]);
        }
    }
    return ((acc[0] + acc[4]) + (acc[1] + acc[5])) + ((acc[2] + acc[6]) + (acc[3] + acc[7]));
}

int oracle_q6k_gemv_x86(size_t n_out, size_t n_in, const float *x, const void *w_q6k, float *y) {
    /* kernel_q6k_gemv.c:159-179 */
    const size_t n_super = n_in / 256;
    if (n_super == 0 || n_super > 64 || n_in % 256 != 0)
        return 1; /* the reference's caller falls back */
    float   d_act[64];
    int8_t  qs[64 * 256];
    int16_t bsums[64 * 16];
    oracle_q8k_quantize(n_super, x, d_act, qs, bsums);
#pragma omp parallel for schedule(static)
    for (size_t r = 0; r < n_out; r++)
        y[r] = oracle_dot_q6k_q8k(n_super, (const uint8_t *) w_q6k + r * n_super * 210, d_act, qs, bsums);
    return 0;
}

/* ---- the x86 backend's batch kernel over a Q6_K table ------------------------------------------
 * cpu_x86_linear_q6k_mN (src/backends/cpu_x86/linear_q6k.c:234-300) over the copy that
 * cpu_x86_linear_q6k_resolve (:84-156) makes at load: q6k_to_w8a8_row (q6k_to_w8a8.c:26-68) keeps
 * the six-bit values q = 0..63 as bytes in element order and, per group of sixteen, the scale
 * ws = d * (float) scale (binary32) and the offset wo = ws * 32. Every activation row is quantised
 * by quantize_x_int8_sym (src/formats/gguf/common.c:204-250: ONE scale per row, amax / 127, 1 when
 * that is zero; lrintf) and summed per sixteen (linear_q6k.c:271-279). Per output and group the
 * integer d = sum of q * a; then
 *   lanes != 0  w8x8_gemm / w8x16_gemm (kernel_w8a8_avx512_vnni.c:176-297), which a host with
 *               AVX-512 VNNI takes for tables of a multiple of 8 rows: acc = fmaf(ws, (float) d,
 *               acc); acc = fmaf(-wo, (float) sum_a, acc), group after group;
 *   lanes == 0  w8a8_dot_scalar (kernel_w8a8_scalar.c:14-34) and the VNNI kernel for other tables
 *               (kernel_w8a8_avx512_vnni.c:90-160), which write acc += ws * (float) d - wo * (float)
 *               sum_a: restated without contraction, every operation rounded, as the reference's
 *               strict build compiles it;
 * and y = scale_x * acc. The interleaving of w8x8_repack / w8x16_repack only places eight or
 * sixteen rows in the lanes of a vector. */

void oracle_q8_sym_row_quantize(size_t n, const float *x, float *scale_out, int8_t *q_out,
                                int32_t *sum16_out) {
    float amax = 0.0f;
    for (size_t i = 0; i < n; i++) {
        const float a = fabsf(x[i]);
        if (a > amax)
            amax = a;
    }
    float scale = amax / 127.0f;
    if (scale == 0.0f)
        scale = 1.0f;
    const float inv = 1.0f / scale;
    for (size_t i = 0; i < n; i++)
        q_out[i] = (int8_t) lrintf(x[i] * inv);
    for (size_t g = 0; g < n / 16; g++) {
        int32_t t = 0;
        for (int i = 0; i < 16; i++)
            t += q_out[16 * g + i];
        sum16_out[g] = t;
    }
    *scale_out = scale;
}

static float oracle_dot_q6k_w8a8(size_t n_super, const uint8_t *row, float scale_x, const int8_t *a,
                                 const int32_t *sum16, int lanes) {
    float acc = 0.0f;
    for (size_t b = 0; b < n_super; b++, row += 210, a += 256, sum16 += 16) {
        const uint8_t *ql = row, *qh = row + 128;
        const int8_t  *sc = (const int8_t *) (row + 192);
        const float    d  = oracle_f16_to_f32((uint16_t) (row[208] | (row[209] << 8)));
        int32_t        dot[16] = {0};
        for (int h = 0; h < 2; h++)
            for (int j = 0; j < 4; j++)
                for (int l = 0; l < 32; l++) {
                    const uint8_t lo = ql[64 * h + 32 * (j & 1) + l];
                    const int     q  = ((j >> 1) ? lo >> 4 : lo & 0xF) |
                                  (((qh[32 * h + l] >> (2 * j)) & 3) << 4);
                    const int e = 128 * h + 32 * j + l;
                    dot[e / 16] += q * a[e];
                }
        for (int k = 0; k < 16; k++) {
            const float ws = d * (float) sc[k];
            const float wo = ws * 32.0f;
            if (lanes) {
                acc = fmaf(ws, (float) dot[k], acc);
                acc = fmaf(-wo, (float) sum16[k], acc);
            } else {
                const float t1 = ws * (float) dot[k];
                const float t2 = wo * (float) sum16[k];
                const float t  = t1 - t2;
                acc            = acc + t;
            }
        }
    }
    return scale_x * acc;
}

int oracle_q6k_linear_x86(size_t m, size_t n_out, size_t n_in, const float *x, const void *w_q6k,
                          float *y, int vnni) {
    if (n_in % 256 != 0 || n_in == 0 || m == 0)
        return -1;
    if (m == 1) /* cpu_x86_linear_q6k_m1: the decode kernel over the table as it lies */
        return oracle_q6k_gemv_x86(n_out, n_in, x, w_q6k, y);
    const int lanes = vnni && n_out % 8 == 0; /* q6k_use_w8x8, linear_q6k.c:61-63 */
    int8_t   *q     = malloc(n_in);
    int32_t  *sum16 = malloc(n_in / 16 * sizeof(int32_t));
    if (!q || !sum16) {
        free(q);
        free(sum16);
        return -2;
    }
    for (size_t i = 0; i < m; i++) {
        float scale_x;
        oracle_q8_sym_row_quantize(n_in, x + i * n_in, &scale_x, q, sum16);
#pragma omp parallel for schedule(static)
        for (size_t r = 0; r < n_out; r++)
            y[i * n_out + r] = oracle_dot_q6k_w8a8(
                n_in / 256, (const uint8_t *) w_q6k + r * (n_in / 256) * 210, scale_x, q, sum16, lanes);
    }
    free(q);
    free(sum16);
    return 0;
}

/* ---- the x86 backend's decode kernel over a Q4_K table ------------------------------------
 * q4kx8_gemv_m1 (src/backends/cpu_x86/kernel_q4kx8_gemm_avx512.c:380-399) over the table that
 * q4k_to_q4kx8_matrix (q4k_to_q4kx8.c:24-115) interleaves eight rows at a time. The interleaving
 * only places the rows' bytes where the eight lanes of the vector kernel find them: each output
 * row's arithmetic involves that row's blocks alone, and it is restated here row by row. */

void oracle_q8k_row_quantize(size_t n_super, const float *x, float *d_out, int8_t *qs_out,
                             int16_t *bsums_out) {
    /* quantize_q8k_row, kernel_q4kx8_gemm_avx512.c:47-77: ONE scale for the whole row,
     * round half away from zero by truncation, clamp, sums per sixteen */
    float amax = 0.0f;
    for (size_t k = 0; k < n_super * 256; k++) {
        const float a  = x[k];
        const float ax = a < 0.0f ? -a : a;
        if (ax > amax)
            amax = ax;
    }
    const float scale = amax == 0.0f ? 1.0f : amax / 127.0f;
    const float inv   = 1.0f / scale;
    *d_out            = scale;
    for (size_t k = 0; k < n_super * 256; k++) {
        const float v = x[k] * inv;
        const int   q = (int) (v < 0.0f ? v - 0.5f : v + 0.5f);
        qs_out[k]     = (int8_t) (q < -128 ? -128 : q > 127 ? 127 : q);
    }
    for (size_t g = 0; g < n_super * 16; g++) {
        int s = 0;
        for (int i = 0; i < 16; i++)
            s += qs_out[g * 16 + i];
        bsums_out[g] = (int16_t) s;
    }
}

/* One row: q4kx8_gemv_one_row_tile (kernel_q4kx8_gemm_avx512.c:81-304) for one of its eight
 * lanes. Per super-block the products of the 4-bit values with the int8 activations are summed
 * as integers per sub-block of 32 and weighted with the sub-block's 6-bit scale; the minima are
 * weighted with the activations' sums per sub-block; each of the two integers joins a binary32
 * accumulator by one fused multiply-add with (d * d_act) and (dmin * d_act) -- both products
 * rounded to binary32 first --, and the result is the difference of the two accumulators. */
static float oracle_dot_q4k_q8k(size_t n_super, const uint8_t *row, float d_act, const int8_t *qs,
                                const int16_t *bsums, int per_pair) {
    float acc = 0.0f, acc_min = 0.0f;
    for (size_t b = 0; b < n_super; b++, row += 144) {
        const float    d    = oracle_f16_to_f32((uint16_t) (row[0] | (row[1] << 8)));
        const float    dmin = oracle_f16_to_f32((uint16_t) (row[2] | (row[3] << 8)));
        const uint8_t *sc = row + 4, *q = row + 16;
        const int8_t  *a  = qs + b * 256;
        int32_t        iacc = 0, iacc_min = 0;
        for (int j = 0; j < 8; j++) { /* sub-block j: elements 32 j .. 32 j + 31 */
            int scale, min;          /* get_scale_min_k4(j), src/formats/gguf/q4_K.c */
            if (j < 4) {
                scale = sc[j] & 63;
                min   = sc[j + 4] & 63;
            } else {
                scale = (sc[j + 4] & 0xF) | ((sc[j - 4] >> 6) << 4);
                min   = (sc[j + 4] >> 4) | ((sc[j] >> 6) << 4);
            }
            int32_t dot = 0;
            for (int l = 0; l < 32; l++) {
                const int v = (j & 1) ? q[32 * (j >> 1) + l] >> 4 : q[32 * (j >> 1) + l] & 0xF;
                dot += v * a[32 * j + l];
            }
            iacc += scale * dot;
            iacc_min += min * (bsums[b * 16 + 2 * j] + bsums[b * 16 + 2 * j + 1]);
            if (per_pair && (j & 1)) {
                /* the 16 x 16 tiles of kernel_q4kx8_gemm_avx512_full.c:94-779 join the
                 * accumulators once per pair of sub-blocks, not once per super-block */
                acc      = fmaf((float) iacc, d * d_act, acc);
                acc_min  = fmaf((float) iacc_min, dmin * d_act, acc_min);
                iacc     = 0;
                iacc_min = 0;
            }
        }
        if (per_pair)
            continue;
        acc     = fmaf((float) iacc, d * d_act, acc);
        acc_min = fmaf((float) iacc_min, dmin * d_act, acc_min);
    }
    return acc - acc_min;
}

int oracle_q4k_gemv_x86(size_t n_out, size_t n_in, const float *x, const void *w_q4k, float *y) {
    const size_t n_super = n_in / 256;
    if (n_in % 256 != 0 || n_super == 0 || n_super > 64 || n_out % 8 != 0)
        return -1; /* shapes the reference's kernel does not take */
    float    d_act;
    int8_t  *qs    = malloc(n_in);
    int16_t *bsums = malloc(n_super * 16 * sizeof(int16_t));
    if (!qs || !bsums) {
        free(qs);
        free(bsums);
        return -2;
    }
    oracle_q8k_row_quantize(n_super, x, &d_act, qs, bsums);
#pragma omp parallel for schedule(static)
    for (size_t r = 0; r < n_out; r++)
        y[r] = oracle_dot_q4k_q8k(n_super, (const uint8_t *) w_q4k + r * n_super * 144, d_act, qs, bsums, 0);
    free(qs);
    free(bsums);
    return 0;
}

/* ---- the x86 backend's batch kernel over a Q4_K table ----------------------------------------
 * cpu_x86_linear_q4k_mN (src/backends/cpu_x86/linear_q4k.c:198-250). A batch whose row count is
 * not a multiple of 4 is the decode kernel row by row (:222-229). Otherwise the rows are quantised
 * four at a time by quantize_q8_Kx4 (q8_kx4.c:21-105) and go through q4kx8_gemm_avx512
 * (kernel_q4kx8_gemm_avx512_full.c:800-860): the 16 x 16 tiles of an AVX-512 host for row counts
 * that are multiples of 16, q4kx8_gemv_avx2_fallback (kernel_q4kx8_gemm_avx512.c:317-371) for the
 * others and on hosts without AVX-512. The fallback is the decode kernel's arithmetic per output
 * (it calls the same q4kx8_gemv_one_row_tile), so its rows differ from the decode kernel's only
 * through the quantiser: still ONE scale per row, but lrintf (ties to even) and no clamp. The
 * tiles form the same integers but join them to the binary32 accumulators once per pair of
 * sub-blocks (full.c:94, 729-778), four times per super-block. */

void oracle_q8kx4_row_quantize(size_t n_super, const float *x, float *d_out, int8_t *qs_out,
                               int16_t *bsums_out) {
    /* quantize_q8_Kx4 for one of its four rows, the int8 values back in element order (the
     * interleaving in stripes of eight only places them for the vector kernel) */
    float amax = 0.0f;
    for (size_t k = 0; k < n_super * 256; k++) {
        const float a = fabsf(x[k]);
        if (a > amax)
            amax = a;
    }
    const float scale = amax == 0.0f ? 1.0f : amax / 127.0f;
    const float inv   = 1.0f / scale;
    *d_out            = scale;
    for (size_t k = 0; k < n_super * 256; k++)
        qs_out[k] = (int8_t) lrintf(x[k] * inv);
    for (size_t g = 0; g < n_super * 16; g++) {
        int s = 0;
        for (int i = 0; i < 16; i++)
            s += qs_out[g * 16 + i];
        bsums_out[g] = (int16_t) s;
    }
}

int oracle_q4k_linear_x86(size_t m, size_t n_out, size_t n_in, const float *x, const void *w_q4k,
                          float *y, int avx512) {
    const size_t n_super = n_in / 256;
    if (n_in % 256 != 0 || n_super == 0 || n_super > 64 || n_out % 8 != 0 || m == 0)
        return -1; /* shapes these kernels do not take */
    const int kx4   = m > 1 && m % 4 == 0;
    /* full.c:831-835: the tiles need both counts to be multiples of 16, and an AVX-512 host */
    const int tiles = avx512 && kx4 && m % 16 == 0 && n_out % 16 == 0;
    int8_t   *qs    = malloc(n_in);
    int16_t  *bsums = malloc(n_super * 16 * sizeof(int16_t));
    if (!qs || !bsums) {
        free(qs);
        free(bsums);
        return -2;
    }
    for (size_t i = 0; i < m; i++) {
        float d_act;
        if (kx4)
            oracle_q8kx4_row_quantize(n_super, x + i * n_in, &d_act, qs, bsums);
        else
            oracle_q8k_row_quantize(n_super, x + i * n_in, &d_act, qs, bsums);
#pragma omp parallel for schedule(static)
        for (size_t r = 0; r < n_out; r++)
            y[i * n_out + r] = oracle_dot_q4k_q8k(
                n_super, (const uint8_t *) w_q4k + r * n_super * 144, d_act, qs, bsums, tiles);
    }
    free(qs);
    free(bsums);
    return 0;
}

void oracle_dequant_q4_K_row(const void *blocks, float *out, size_t n_elems) {
    /* q4_K.c:18-49; the block layout of src/quant/quant_blocks.h:50-56 by offsets */
    const uint8_t *p = (const uint8_t *) blocks;
    for (size_t b = 0; b < n_elems / 256; b++, p += 144) {
        const float    d    = oracle_f16_to_f32((uint16_t) (p[0] | (p[1] << 8)));
        const float    dmin = oracle_f16_to_f32((uint16_t) (p[2] | (p[3] << 8)));
        const uint8_t *sc = p + 4, *q = p + 16;
        float         *y  = out + b * 256;
        for (int s = 0; s < 4; s++, q += 32) {
            uint8_t scale[2], min[2];
            for (int t = 0; t < 2; t++) { /* get_scale_min_k4(2 s + t) */
                const int j = 2 * s + t;
                if (j < 4) {
                    scale[t] = sc[j] & 63;
                    min[t]   = sc[j + 4] & 63;
                } else {
                    scale[t] = (uint8_t) ((sc[j + 4] & 0xF) | ((sc[j - 4] >> 6) << 4));
                    min[t]   = (uint8_t) ((sc[j + 4] >> 4) | ((sc[j] >> 6) << 4));
                }
            }
            const float d1 = d * (float) scale[0], m1 = dmin * (float) min[0];
            const float d2 = d * (float) scale[1], m2 = dmin * (float) min[1];
            for (int l = 0; l < 32; l++) {
                const float a = d1 * (float) (q[l] & 0xF);
                y[64 * s + l] = a - m1;
            }
            for (int l = 0; l < 32; l++) {
                const float a      = d2 * (float) (q[l] >> 4);
                y[64 * s + 32 + l] = a - m2;
            }
        }
    }
}

void oracle_q4k_linear_f64(size_t m, size_t n_out, size_t n_in, const float *x,
                           const void *w_q4k, float *y) {
    const size_t row_bytes = n_in / 256 * 144;
#pragma omp parallel
    {
        float *row = (float *) malloc(n_in * sizeof(float));
#pragma omp for schedule(static)
        for (size_t j = 0; j < n_out; j++) {
            oracle_dequant_q4_K_row((const uint8_t *) w_q4k + j * row_bytes, row, n_in);
            for (size_t i = 0; i < m; i++) {
                double acc = 0.0;
                for (size_t k = 0; k < n_in; k++)
                    acc += (double) x[i * n_in + k] * (double) row[k];
                y[i * n_out + j] = (float) acc;
            }
        }
        free(row);
    }
}
