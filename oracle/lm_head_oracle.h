/*
 * lm_head_oracle.h -- TEST INFRASTRUCTURE, not part of the shipped library: a scalar CPU
 * restatement of the two steps the reference runs between the last layer and the sampler
 * (src/archs/transformer/forward/head.c:94-129): the output RMS norm and the tied lm_head
 * projection for F16 weights. Only tests/, the smoke check and the cpu_baseline leg of bench.py
 * may load it.
 *
 * Pinned by: the reference's own kernel compiled from its tree (oracle/_ref/libgeist_ref_f16gemv
 * .so, src/backends/cpu_x86/kernel_f16_gemv.c) bit for bit on random and adversarial inputs
 * (tests/test_lm_head_oracle.py); the exact-double reference of the reference's unit test
 * (tests/test_q8w_gemv_unit.c:49-56) within the bound of fp32 accumulation; closed forms for the
 * norm (constant rows, unit weights) and numpy in float64.
 */
#ifndef GEIST_LM_HEAD_ORACLE_H
#define GEIST_LM_HEAD_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* IEEE binary16 -> binary32, exact (src/formats/gguf/common.c:29-62). */
float oracle_f16_to_f32(uint16_t h);
/* binary32 -> binary16, round to nearest even (what tests/test_q8w_gemv_unit.c:24-26 gets from
 * F16C); used to build test weights. */
uint16_t oracle_f32_to_f16(float v);

/* y[r] = sum_i f16_to_f32(W[r,i]) * x[i] in the summation order of f16_gemv_m1
 * (src/backends/cpu_x86/kernel_f16_gemv.c:34-64): sixteen chains of fused multiply-adds --
 * chain j takes the elements 16 t + j in order of t; a trailing block of eight extends chains
 * 0..7 --, then (chain j + chain j+8), then (lane i + lane i+4), then ((0+1) + (2+3)), then the
 * elements of an n_in % 8 tail one by one. */
void oracle_f16_gemv_m1(size_t n_out, size_t n_in, const float *x, const uint16_t *w_f16, float *y);

/* The int8 form of the table. f16_to_q8w (kernel_f16_gemv.c:66-93): scales[r] = max|w| / 127,
 * wq = clamp(lrintf(w * (127 / max|w|)), -127, 127), a row of zeros gets scale 0 and zeros.
 * q8w_gemv_m1 (kernel_f16_gemv.c:95-127): the chains and tree of f16_gemv_m1 over (float) wq,
 * then times scales[r]. */
void oracle_f16_to_q8w(size_t n_out, size_t n_in, const uint16_t *w_f16, int8_t *wq, float *scales);
void oracle_q8w_gemv_m1(size_t n_out, size_t n_in, const float *x, const int8_t *wq,
                        const float *scales, float *y);

/* The portable kernel, which the x86 backend also runs for more than one activation row
 * (cpu_scalar_w_quant_m1 / _mN, src/backends/cpu_scalar/weight_resolve.c:186-241, for F16
 * weights): y[i][j] = (float) sum_k (double) x[i][k] * (double) f16(W[j][k]), the sum in double in
 * index order. (The products are exact in double, so a fused multiply-add gives the same bits.)
 * Pinned by numpy's float64 dot wherever that is not within the sums' error of a binary32
 * rounding boundary, and by exactly representable cases. */
void oracle_f16_linear_f64(size_t m, size_t n_out, size_t n_in, const float *x,
                           const uint16_t *w_f16, float *y);

/* Q6_K weights: super-blocks of 256 elements in 210 bytes -- ql[128] (low 4 bits), qh[64] (high
 * 2 bits), scales[16] (int8, one per 16 elements), d (binary16) -- src/quant/quant_blocks.h:67-73.
 * dequant_q6_K_row (src/formats/gguf/q6_K.c:13-45): element 128 h + 32 j + l of a block
 * (h < 2, j < 4, l < 32) is d * scales[8 h + 2 j + l / 16] * (q - 32) with
 * q = nibble (j >> 1) of ql[64 h + 32 (j & 1) + l] | ((qh[32 h + l] >> 2 j) & 3) << 4,
 * multiplied left to right in binary32. (Both products are exact: 11 + 8 + 6 significant bits.)
 * n_elems a multiple of 256. */
void oracle_dequant_q6_K_row(const void *blocks, float *out, size_t n_elems);
/* cpu_scalar_w_quant_m1 / _mN over a Q6_K table (src/backends/cpu_scalar/weight_resolve.c:
 * 186-241 with the Q6_K case of dequant_one_row_for, :86-88): row j of the table is
 * n_in / 256 blocks; y[i][j] = (float) sum_k (double) x[i][k] * (double) w[j][k], the sum in
 * double in index order. Pinned by the reference's own weight_resolve.c and q6_K.c compiled from
 * its tree (oracle/_ref/libgeist_ref_wquant.so, tests/test_q6k_oracle.py) bit for bit, and by
 * golden vectors written from that build. */
void oracle_q6k_linear_f64(size_t m, size_t n_out, size_t n_in, const float *x,
                           const void *w_q6k, float *y);

/* What the reference's x86 backend decodes a Q6_K table with when it has the raw table (one
 * row: cpu_x86_linear_q6k_m1, src/backends/cpu_x86/linear_q6k.c:187-208 -> q6k_gemv_m1,
 * kernel_q6k_gemv.c:159-179): the activation row quantised per super-block of 256 to int8
 * (d = amax / 127, q = lrintf(x * (127 / amax)), sums per sixteen; kernel_q6k_gemv.c:43-67),
 * integer dot products, and per super-block one fused multiply-add per lane of an eight-lane
 * binary32 accumulator (kernel_q6k_gemv.c:90-157), the lanes added as hsum_ps_avx adds them.
 * Returns 1 where the reference's kernel returns without a result (n_in / 256 outside 1 .. 64).
 * Pinned bit for bit by that translation unit compiled from the reference's tree
 * (tests/test_q6k_x86_oracle.py) and by golden vectors written from it. */
void oracle_q8k_quantize(size_t n_super, const float *x, float *d_out, int8_t *qs_out,
                         int16_t *bsums_out);
int  oracle_q6k_gemv_x86(size_t n_out, size_t n_in, const float *x, const void *w_q6k, float *y);
/* The x86 backend's projection of a batch over a Q6_K table (cpu_x86_linear_q6k_mN,
 * src/backends/cpu_x86/linear_q6k.c:234-300, over the int8 copy of cpu_x86_linear_q6k_resolve):
 * the rows quantised with one scale each (quantize_x_int8_sym), integer dot products per group
 * of sixteen, binary32 accumulation group after group -- with vnni != 0 and a table of a multiple
 * of 8 rows by two fused multiply-adds per group (w8x8_gemm / w8x16_gemm), otherwise by the
 * rounded expression of w8a8_dot_scalar. One row is the decode kernel. x [m, n_in], y [m, n_out].
 * Pinned to those translation units compiled from the reference's tree
 * (tests/test_q6k_x86_oracle.py). */
void oracle_q8_sym_row_quantize(size_t n, const float *x, float *scale_out, int8_t *q_out,
                                int32_t *sum16_out);
int  oracle_q6k_linear_x86(size_t m, size_t n_out, size_t n_in, const float *x, const void *w_q6k,
                           float *y, int vnni);

/* The x86 backend's decode kernel over a Q4_K table (q4kx8_gemv_m1,
 * src/backends/cpu_x86/kernel_q4kx8_gemm_avx512.c:47-77 the activation quantiser -- one scale for
 * the whole row, round half away from zero --, :81-304 the dot products), restated row by row.
 * n_out a multiple of 8 and n_in / 256 <= 64, as the reference's kernel requires (-1 otherwise).
 * oracle_q8k_row_quantize: d_out one float, qs_out n_super * 256 int8, bsums_out n_super * 16. */
void oracle_q8k_row_quantize(size_t n_super, const float *x, float *d_out, int8_t *qs_out,
                             int16_t *bsums_out);
int oracle_q4k_gemv_x86(size_t n_out, size_t n_in, const float *x, const void *w_q4k, float *y);
/* The x86 backend's batch kernel over a Q4_K table (cpu_x86_linear_q4k_mN,
 * src/backends/cpu_x86/linear_q4k.c:198-250): row counts that are no multiple of 4 are the decode
 * kernel row by row; the others are quantised by quantize_q8_Kx4 (q8_kx4.c:21-105: one scale per
 * row, lrintf) and multiplied by q4kx8_gemm_avx512: per output the decode kernel's arithmetic,
 * except that with avx512 != 0 (a host with AVX-512) row counts that are multiples of 16 over a
 * table of a multiple of 16 rows go through 16 x 16 tiles, which join the binary32 accumulators
 * once per pair of sub-blocks. x [m, n_in], y [m, n_out]. Pinned to those translation units compiled from the
 * reference's tree (tests/test_q4k_x86_oracle.py), the 16 x 16 AVX-512 tiles included. */
void oracle_q8kx4_row_quantize(size_t n_super, const float *x, float *d_out, int8_t *qs_out,
                               int16_t *bsums_out);
int oracle_q4k_linear_x86(size_t m, size_t n_out, size_t n_in, const float *x, const void *w_q4k,
                          float *y, int avx512);

/* The same pair for a Q4_K table (super-blocks of 144 bytes: d, dmin in binary16, eight 6-bit
 * scales and eight 6-bit minima packed into 12 bytes, 128 bytes of 4-bit values;
 * src/quant/quant_blocks.h:50-56). dequant_q4_K_row (src/formats/gguf/q4_K.c:18-49, scales by
 * get_scale_min_k4, quant_blocks.h:103-111): element 64 s + l of a block is
 * (d * sc[2s]) * (qs[32 s + l] & 15) - dmin * m[2s], element 64 s + 32 + l the same with the
 * high nibble and sc / m[2s + 1], each step rounded to binary32 (the product with the 4-bit value
 * is exact, so a fused multiply-subtract gives the same bits). The projection is
 * cpu_scalar_w_quant_m1 / _mN as above. Pinned bit for bit by the reference's files compiled from
 * its tree (tests/test_q4k_oracle.py) and by hand-built blocks. */
void oracle_dequant_q4_K_row(const void *blocks, float *out, size_t n_elems);
void oracle_q4k_linear_f64(size_t m, size_t n_out, size_t n_in, const float *x,
                           const void *w_q4k, float *y);

/* y = x * weight * rsqrt(mean(x^2) + eps) per row (cpu_scalar_rmsnorm,
 * src/backends/cpu_scalar/elementwise.c:241-280): sum of squares in double in index order,
 * inv = (float)(1.0 / sqrt(sum / n + (double) eps)), y_i = (x_i * inv) * w_i in binary32. */
void oracle_rmsnorm_rows(size_t n_rows, size_t n, const float *x, const float *w, float eps,
                         float *y);

#ifdef __cplusplus
}
#endif
#endif
