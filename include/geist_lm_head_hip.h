/*
 * geist_lm_head_hip.h -- the output head in front of the sampler, on the device: the RMS norm and
 * the tied F16 lm_head projection of the reference's finalize step
 * (src/archs/transformer/forward/head.c:94-129). With them the logits are written by the GPU
 * into the buffer the sampler reads (include/geist_sampler_hip.h); nothing of vocabulary size
 * crosses to the host. Both functions enqueue on the sampler's stream and reproduce the
 * reference's CPU results bit for bit.
 */
#ifndef GEIST_LM_HEAD_HIP_H
#define GEIST_LM_HEAD_HIP_H

#include "geist_sampler_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Replaces prims->rmsnorm as head.c:99-101 calls it (cpu_scalar_rmsnorm,
 * src/backends/cpu_scalar/elementwise.c:241-280): for each of n_rows rows of n floats,
 *   inv = (float)(1.0 / sqrt(sum_i (double)x_i^2 / n + (double)eps)),  y_i = (x_i * inv) * w_i.
 * Row r of x starts at d_x + r * ld_x, of y at d_y + r * ld_y; d_y may be d_x. */
int geist_hip_rmsnorm_rows(geist_hip_sampler *s, const float *d_x, size_t ld_x,
                           const float *d_weight, float eps, size_t n_rows, size_t n, float *d_y,
                           size_t ld_y);

/* Replaces f16_gemv_m1 (src/backends/cpu_x86/kernel_f16_gemv.h:22-25, kernel_f16_gemv.c:34-64;
 * bound as linear_m1 of an F16 weight at src/backends/cpu_x86/backend.c:318-324, 406-411), the
 * kernel behind the tied F16 lm_head at head.c:114-126:
 *   d_y[m * ld_y + r] = sum_i f16_to_f32(d_w_f16[r * n_in + i]) * d_x[m * ld_x + i]
 * for every activation row m < n_rows, with the reference's order of summation (sixteen chains
 * of fused multiply-adds folded in a fixed tree), so each row equals what f16_gemv_m1 returns
 * for it. The weights are read once for up to 8 activation rows. n_in must be a multiple of 8
 * (GEIST_HIP_E_UNSUPPORTED otherwise: the reference adds a remainder element by element, with
 * rounding that depends on how it was compiled); d_w_f16 must be 16-byte aligned. */
int geist_hip_f16_gemv_rows(geist_hip_sampler *s, const uint16_t *d_w_f16, size_t n_out,
                            size_t n_in, const float *d_x, size_t ld_x, size_t n_rows, float *d_y,
                            size_t ld_y);

/* geist_hip_f16_linear_rows replaces the portable kernel cpu_scalar_w_quant_m1 / _mN for F16
 * weights (src/backends/cpu_scalar/weight_resolve.c:186-241), which is also what the x86 backend
 * runs for more than one activation row (its F16 and int8 kernels are decode-only, linear_m1):
 *   d_y[m * ld_y + r] = (float) sum_i (double) d_x[m * ld_x + i] * (double) f16(W[r][i])
 * with the sum in double in index order, bit for bit: the device adds in another order and
 * repeats, in the reference's order, the few sums that lie close enough to a binary32 rounding
 * boundary for the order to matter. Same argument rules as geist_hip_f16_gemv_rows. The kernels
 * use a buffer in the sampler (the activations in double, the list of outputs to repeat):
 * geist_hip_f16_linear_reserve sizes it for weights of up to n_out x n_in at set-up, where the
 * reference sizes its scratch (forward/step.c:398-409); a call for a larger shape than was
 * reserved sizes it again, with a device synchronisation. */
int geist_hip_f16_linear_reserve(geist_hip_sampler *s, size_t n_out, size_t n_in);
int geist_hip_f16_linear_rows(geist_hip_sampler *s, const uint16_t *d_w_f16, size_t n_out,
                              size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                              float *d_y, size_t ld_y);

/* Which of the reference's backends the projection inside geist_hip_project_sample_rows (and
 * the head's project_finalize calls) stands for:
 *   GEIST_HIP_PROJECTION_X86       one row: f16_gemv_m1, over a Q6_K table q6k_gemv_m1, over a
 *                                  packed Q4_K table q4kx8_gemv_m1; more rows: over a Q6_K table
 *                                  cpu_x86_linear_q6k_mN and over a packed Q4_K table
 *                                  cpu_x86_linear_q4k_mN, as a host with AVX-512 (VNNI) runs
 *                                  them, over the F16 table and its int8 form the portable
 *                                  kernel (default)
 *   GEIST_HIP_PROJECTION_PORTABLE  the portable kernel for any number of rows, as on the
 *                                  reference's cpu_scalar backend (weight_resolve.c:247-252 sets
 *                                  linear_m1 and linear_mN alike)
 *   GEIST_HIP_PROJECTION_X86_AVX2  as _X86, for a host without AVX-512 (or one run with
 *                                  GEIST_FORCE_ISA=avx2). Two differences: a Q4_K batch of a
 *                                  multiple of 16 rows goes through the AVX2 kernel instead of
 *                                  the 16 x 16 tiles (kernel_q4kx8_gemm_avx512_full.c:816-835),
 *                                  and a Q6_K batch through the scalar W8A8 kernel instead of
 *                                  the lane kernels (linear_q6k.c:61-63, 281-295) */
#define GEIST_HIP_PROJECTION_X86 0
#define GEIST_HIP_PROJECTION_PORTABLE 1
#define GEIST_HIP_PROJECTION_X86_AVX2 2
int geist_hip_sampler_set_projection(geist_hip_sampler *s, int mode);

/* The int8 form of the tied table, which the reference's x86 backend uses for the lm_head unless
 * GEIST_Q8_LMHEAD=0 (src/backends/cpu_x86/backend.c:344-372): half the bytes per decode step.
 *
 * geist_hip_f16_to_q8w replaces f16_to_q8w (kernel_f16_gemv.c:66-93), run once at load:
 *   scales[r] = max_k |w[r][k]| / 127,  wq[r][k] = clamp(lrintf(w[r][k] * (127 / max|w[r]|)), +-127)
 * with IEEE divisions (the reference's release build compiles with -ffast-math, which may form
 * the first quotient by a reciprocal; its strict build is matched bit for bit).
 * geist_hip_q8w_gemv_rows replaces q8w_gemv_m1 (kernel_f16_gemv.c:95-127):
 *   d_y[m * ld_y + r] = (sum_i (float)wq[r][i] * d_x[m * ld_x + i]) * scales[r]
 * in the reference's order of summation (the chains and the tree of f16_gemv_m1), bit for bit.
 * n_in must be a multiple of 16, d_wq 16-byte aligned. */
int geist_hip_f16_to_q8w(geist_hip_sampler *s, const uint16_t *d_w_f16, size_t n_out, size_t n_in,
                         int8_t *d_wq, float *d_scales);
int geist_hip_q8w_gemv_rows(geist_hip_sampler *s, const int8_t *d_wq, const float *d_scales,
                            size_t n_out, size_t n_in, const float *d_x, size_t ld_x,
                            size_t n_rows, float *d_y, size_t ld_y);

/* The tail of a forward pass in one call (head.c:94-188 / 224-304): norm, projection, sampling
 * of `rows` hidden rows. Equal in results to geist_hip_rmsnorm_rows, the projection and
 * geist_hip_sample_rows[_rng] on d_logits. The projection is the one the reference's x86 backend
 * runs: for one row its decode kernel (geist_hip_f16_gemv_rows), for more rows the portable
 * kernel (geist_hip_f16_linear_rows; the x86 kernels are linear_m1 only,
 * src/archs/transformer/forward/linear.c:34-56). For one row whose configuration takes the
 * top-k path without a soft-cap, the projection also leaves the per-thread maxima the sampler's
 * first pass would compute, and that pass is skipped.
 *   d_normed   [rows, d_model] receives the normed rows
 *   d_logits   [rows, ld_logits] receives the logits (row stride ld_logits >= n_vocab)
 *   d_uniforms one draw per row, or NULL with d_rng_states != NULL: xorshift64* states as in
 *              geist_hip_sample_rows_rng (`shared` as there); both NULL only for greedy params
 * rows <= max_rows and n_vocab <= max_vocab of the sampler. */
int geist_hip_project_sample_rows(geist_hip_sampler *s, const float *d_hidden, size_t ld_hidden,
                                  size_t rows, size_t d_model, const float *d_norm_weight,
                                  float rms_eps, const uint16_t *d_embed_f16, size_t n_vocab,
                                  float *d_normed, float *d_logits, size_t ld_logits,
                                  const struct geist_hip_sample_params *params,
                                  const float *d_uniforms, uint64_t *d_rng_states, int shared,
                                  geist_hip_token_t *d_out_tokens);

/* The same tail over the int8 form of the table (the reference's default for a decode step on
 * x86, src/backends/cpu_x86/backend.c:332-342 behind head.c:114-126): d_embed_q8 [n_vocab,
 * d_model] and d_scales [n_vocab] as geist_hip_f16_to_q8w writes them; d_model a multiple of 16.
 * Equal in results to geist_hip_rmsnorm_rows + geist_hip_q8w_gemv_rows + the sampler, for any
 * number of rows (the reference has the int8 table for one row at a time only). */
int geist_hip_project_sample_rows_q8w(geist_hip_sampler *s, const float *d_hidden,
                                      size_t ld_hidden, size_t rows, size_t d_model,
                                      const float *d_norm_weight, float rms_eps,
                                      const int8_t *d_embed_q8, const float *d_scales,
                                      size_t n_vocab, float *d_normed, float *d_logits,
                                      size_t ld_logits,
                                      const struct geist_hip_sample_params *params,
                                      const float *d_uniforms, uint64_t *d_rng_states, int shared,
                                      geist_hip_token_t *d_out_tokens);

/* The lm_head over a Q6_K table, the tied embedding of the Gemma models (which also carry the
 * soft-cap that the sampler applies): d_w_q6k holds n_out rows of n_in / 256 super-blocks of 210
 * bytes (src/quant/quant_blocks.h:67-73), as they lie in a GGUF file, 4-byte aligned, n_in a
 * multiple of 256 (GEIST_HIP_E_UNSUPPORTED otherwise: the format has no partial blocks).
 * geist_hip_q6k_linear_rows replaces cpu_scalar_w_quant_m1 / _mN for that dtype
 * (src/backends/cpu_scalar/weight_resolve.c:86-88, 186-241; decoder: src/formats/gguf/q6_K.c):
 *   d_y[m * ld_y + r] = (float) sum_k (double) d_x[m * ld_x + k] * (double) w[r][k],
 * w = d * scale * (q - 32) in binary32, the sum in double in index order, bit for bit (the device
 * adds in another order and repeats, in the reference's order, the few sums that lie close enough
 * to a binary32 rounding boundary for the order to matter). This is the arithmetic of the
 * reference's portable backend for any number of rows. Its x86 backend runs other kernels over
 * such a table (cpu_x86_linear_q6k_resolve, src/backends/cpu_x86/backend.c:395-397): for one row
 * the integer decode kernel q6k_gemv_m1, which geist_hip_q6k_packed_gemv_x86_rows below
 * reproduces; for more rows a GEMM over an int8 copy of the table and int8 activations
 * (cpu_x86_linear_q6k_mN, src/backends/cpu_x86/linear_q6k.c:234-300), which is not reproduced:
 * batches get the portable arithmetic. geist_hip_q6k_linear_reserve sizes the scratch ahead of
 * the first call, as geist_hip_f16_linear_reserve does. */
int geist_hip_q6k_linear_reserve(geist_hip_sampler *s, size_t n_out, size_t n_in);
int geist_hip_q6k_linear_rows(geist_hip_sampler *s, const void *d_w_q6k, size_t n_out, size_t n_in,
                              const float *d_x, size_t ld_x, size_t n_rows, float *d_y,
                              size_t ld_y);
/* No counterpart in the reference (its x86 backend likewise re-lays the table at load, into
 * binary32: cpu_x86_linear_q6k_resolve). The same bytes in the order the device reads them, so
 * that the projection streams the table at the rate of the memory: the rows in groups of 64, per
 * group the blocks in order, per block the 53 dwords of the 64 rows with the rows innermost
 * (geistlib_amd/csrc/lm_head_q6k.hip has the exact layout). geist_hip_q6k_packed_bytes: size of
 * the packed copy (1 % above the table's; 0 for a shape the format does not allow).
 * geist_hip_q6k_pack: once per model, d_packed 16-byte aligned. geist_hip_q6k_packed_linear_rows:
 * geist_hip_q6k_linear_rows over the packed copy, same results bit for bit; it adds every row's
 * products in index order itself, so nothing is repeated. */
size_t geist_hip_q6k_packed_bytes(size_t n_out, size_t n_in);
int geist_hip_q6k_pack(geist_hip_sampler *s, const void *d_w_q6k, size_t n_out, size_t n_in,
                       void *d_packed);
int geist_hip_q6k_packed_linear_rows(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                     size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                     float *d_y, size_t ld_y);
/* The x86 backend's decode kernel over the packed copy: replaces q6k_gemv_m1
 * (src/backends/cpu_x86/kernel_q6k_gemv.c:43-157, called from cpu_x86_linear_q6k_m1,
 * src/backends/cpu_x86/linear_q6k.c:205-207), bit for bit. Per super-block of 256 elements the
 * activations become int8 with one scale (amax / 127, round to nearest even), the products with
 * the six-bit weights are summed as integers in eight lanes, each lane's sum joins a binary32
 * accumulator by one fused multiply-add, and the eight accumulators are added as the AVX2
 * horizontal sum adds them. Each activation row is a pass of its own over the table, as each
 * call of the reference's kernel is. Activations must be finite. */
int geist_hip_q6k_packed_gemv_x86_rows(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                       size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                       float *d_y, size_t ld_y);
/* The same over the table as it lies in the file (4-byte aligned), for callers that keep no
 * packed copy: the same results bit for bit, at the price of the table's scattered reads. */
int geist_hip_q6k_gemv_x86_rows(geist_hip_sampler *s, const void *d_w_q6k, size_t n_out,
                                size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                float *d_y, size_t ld_y);
/* The two halves of that kernel for callers that keep the int8 activations (several tables
 * projected from one activation row, or the quantiser placed in an earlier launch):
 * geist_hip_q8k_quantize_rows replaces the activation quantiser of kernel_q6k_gemv.c:43-67 --
 * d_act, 64-byte aligned, geist_hip_q8k_act_bytes(n_in, n_rows) bytes, gets per row and
 * super-block 96 dwords: the 256 activations as int8 in element order, their sixteen sums per
 * group of sixteen as int32, the scale as binary32, padding. geist_hip_q6k_packed_gemv_q8k
 * replaces the dot products of kernel_q6k_gemv.c:90-157 for one row of d_act. */
size_t geist_hip_q8k_act_bytes(size_t n_in, size_t n_rows);
int geist_hip_q8k_quantize_rows(geist_hip_sampler *s, const float *d_x, size_t ld_x, size_t n_rows,
                                size_t n_in, void *d_act);
int geist_hip_q6k_packed_gemv_q8k(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                  size_t n_in, const void *d_act, float *d_y);
/* geist_hip_q6k_packed_linear_x86_rows replaces cpu_x86_linear_q6k_mN
 * (src/backends/cpu_x86/linear_q6k.c:234-300) for n_rows > 1, and the decode kernel for one row,
 * bit for bit. The reference multiplies an int8 copy of the table that it makes at load
 * (cpu_x86_linear_q6k_resolve, :84-156; q6k_to_w8a8_row, q6k_to_w8a8.c:26-68: the six-bit values
 * as bytes, a binary32 scale and offset per group of sixteen) with the rows quantised by
 * quantize_x_int8_sym (src/formats/gguf/common.c:204-250: one scale per row, lrintf): integer dot
 * products per group of sixteen, joined in binary32 group after group. The device needs no such
 * copy: the packed copy holds the same values and scales. How the groups are joined depends on
 * the host, and follows geist_hip_sampler_set_projection: _X86 stands for a host with AVX-512
 * VNNI, whose lane kernels (w8x8_gemm / w8x16_gemm, kernel_w8a8_avx512_vnni.c:176-297: two fused
 * multiply-adds per group) take tables of a multiple of 8 rows; other tables there, and every
 * table in mode _X86_AVX2 (a host without VNNI, or GEIST_FORCE_ISA=avx2), get the expression of
 * w8a8_dot_scalar (kernel_w8a8_scalar.c:14-34) with every operation rounded, as the reference's
 * strict build compiles it. Up to eight rows share a pass over the table. Activations must be
 * finite. */
int geist_hip_q6k_packed_linear_x86_rows(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                         size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                         float *d_y, size_t ld_y);
/* The same over the table as it lies in the file (4-byte aligned): the same results bit for bit. */
int geist_hip_q6k_linear_x86_rows(geist_hip_sampler *s, const void *d_w_q6k, size_t n_out,
                                  size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                  float *d_y, size_t ld_y);
/* The tail of a forward pass over that table: geist_hip_rmsnorm_rows, the projection and the
 * sampler (soft-cap included) in one call, arguments as geist_hip_project_sample_rows. The
 * projection follows geist_hip_sampler_set_projection: in the modes GEIST_HIP_PROJECTION_X86
 * (default) and _X86_AVX2 one row gets the x86 backend's decode kernel
 * (geist_hip_q6k_gemv_x86_rows / geist_hip_q6k_packed_gemv_x86_rows) and a batch its batch path
 * (geist_hip_q6k_linear_x86_rows / geist_hip_q6k_packed_linear_x86_rows); any call in mode
 * _PORTABLE gets the portable arithmetic (geist_hip_q6k_linear_rows /
 * geist_hip_q6k_packed_linear_rows). Over the packed copy and over the table as it lies in the
 * file the logits are the same bit for bit. */
int geist_hip_project_sample_rows_q6k(geist_hip_sampler *s, const float *d_hidden,
                                      size_t ld_hidden, size_t rows, size_t d_model,
                                      const float *d_norm_weight, float rms_eps,
                                      const void *d_embed_q6k, size_t n_vocab, float *d_normed,
                                      float *d_logits, size_t ld_logits,
                                      const struct geist_hip_sample_params *params,
                                      const float *d_uniforms, uint64_t *d_rng_states, int shared,
                                      geist_hip_token_t *d_out_tokens);

int geist_hip_project_sample_rows_q6k_packed(geist_hip_sampler *s, const float *d_hidden,
                                             size_t ld_hidden, size_t rows, size_t d_model,
                                             const float *d_norm_weight, float rms_eps,
                                             const void *d_embed_packed, size_t n_vocab,
                                             float *d_normed, float *d_logits, size_t ld_logits,
                                             const struct geist_hip_sample_params *params,
                                             const float *d_uniforms, uint64_t *d_rng_states,
                                             int shared, geist_hip_token_t *d_out_tokens);

/* A Q4_K table (n_out rows of n_in / 256 super-blocks of 144 bytes: d and dmin in binary16, eight
 * 6-bit scales and minima, 256 four-bit values; src/quant/quant_blocks.h:50-56), packed form
 * only. geist_hip_q4k_packed_bytes: size of the packed copy (148 bytes per block; 0 for a shape
 * that is not supported); geist_hip_q4k_pack: once per model, table 4-byte and d_packed 16-byte
 * aligned; geist_hip_q4k_packed_linear_rows: d_y[i][j] = (float) sum_k (double) d_x[i][k] *
 * (double) w[j][k] in index order, w as dequant_q4_K_row forms it (src/formats/gguf/q4_K.c:18-49)
 * -- cpu_scalar_w_quant_m1 / _mN for that dtype (weight_resolve.c:82-83, 186-241), bit for bit.
 * geist_hip_q6k_linear_reserve sizes the scratch. geist_hip_project_sample_rows_q4k_packed: the
 * tail of a forward pass over the packed table, as geist_hip_project_sample_rows_q6k_packed. */
size_t geist_hip_q4k_packed_bytes(size_t n_out, size_t n_in);
int geist_hip_q4k_pack(geist_hip_sampler *s, const void *d_w_q4k, size_t n_out, size_t n_in,
                       void *d_packed);
int geist_hip_q4k_packed_linear_rows(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                     size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                     float *d_y, size_t ld_y);
/* The x86 backend's decode kernel over the packed copy: replaces q4kx8_gemv_m1
 * (src/backends/cpu_x86/kernel_q4kx8_gemm_avx512.c:47-77, 81-304, 380-399; reached from
 * cpu_x86_linear_q4k_m1, src/backends/cpu_x86/linear_q4k.c:163-166, over the table that
 * q4k_to_q4kx8_matrix interleaves), bit for bit: the activation row becomes int8 with ONE scale
 * (amax / 127, round half away from zero), the products with the 4-bit values are summed as
 * integers per sub-block of 32 and weighted with the sub-block's scale, the minima with the
 * activations' sums; per super-block each of the two integers joins a binary32 accumulator by a
 * fused multiply-add, and the result is the difference of the accumulators. For the shapes that
 * kernel takes -- n_out a multiple of 8, n_in / 256 <= 64 -- and GEIST_HIP_E_UNSUPPORTED for
 * others (the reference sends those through its W4A8 kernels, which are not reproduced). Every
 * row gets the decode kernel's result; up to four rows share a pass over the table. Activations
 * must be finite.
 *
 * geist_hip_q4k_packed_linear_x86_rows replaces cpu_x86_linear_q4k_mN
 * (src/backends/cpu_x86/linear_q4k.c:198-250) for n_rows > 1, and the decode kernel for one row:
 * a row count that is no multiple of 4 is the decode kernel row by row (:222-229); a multiple of
 * 4 is quantised by quantize_q8_Kx4 (q8_kx4.c:21-105: one scale per row, lrintf) and goes
 * through q4kx8_gemm_avx512 (kernel_q4kx8_gemm_avx512_full.c:800-860), whose AVX2 kernel is the
 * decode kernel's arithmetic per output and whose 16 x 16 tiles -- row counts that are
 * multiples of 16 over a table of a multiple of 16 rows, on a host with AVX-512 -- join the
 * binary32 accumulators once per pair of sub-blocks instead of once per super-block. Which host
 * follows geist_hip_sampler_set_projection (_X86: with AVX-512; _X86_AVX2: without). Bit for bit
 * in all three cases.
 *
 * geist_hip_project_sample_rows_q4k_packed follows geist_hip_sampler_set_projection: in the
 * modes _X86 / _X86_AVX2 a table of such a shape gets geist_hip_q4k_packed_linear_x86_rows;
 * other shapes and any call in mode _PORTABLE get geist_hip_q4k_packed_linear_rows. */
int geist_hip_q4k_packed_gemv_x86_rows(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                       size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                       float *d_y, size_t ld_y);
int geist_hip_q4k_packed_linear_x86_rows(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                         size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                         float *d_y, size_t ld_y);
/* The two halves of that kernel, as for Q6_K: geist_hip_q8k_row_quantize replaces the activation
 * quantiser of kernel_q4kx8_gemm_avx512.c:47-77 for one row -- d_act, 64-byte aligned,
 * geist_hip_q8k_row_act_bytes(n_in) bytes, gets per super-block 72 dwords (the 256 activations as
 * int8, per eight elements the even ones and then the odd ones; their eight sums per sub-block
 * of 32 as int32) and behind the last block the row's scale as binary32 and padding --, and
 * geist_hip_q4k_packed_gemv_q8k replaces the dot products of :81-304 over it. */
size_t geist_hip_q8k_row_act_bytes(size_t n_in);
int geist_hip_q8k_row_quantize(geist_hip_sampler *s, const float *d_x, size_t n_in, void *d_act);
int geist_hip_q4k_packed_gemv_q8k(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                  size_t n_in, const void *d_act, float *d_y);
int geist_hip_project_sample_rows_q4k_packed(geist_hip_sampler *s, const float *d_hidden,
                                             size_t ld_hidden, size_t rows, size_t d_model,
                                             const float *d_norm_weight, float rms_eps,
                                             const void *d_embed_packed, size_t n_vocab,
                                             float *d_normed, float *d_logits, size_t ld_logits,
                                             const struct geist_hip_sample_params *params,
                                             const float *d_uniforms, uint64_t *d_rng_states,
                                             int shared, geist_hip_token_t *d_out_tokens);

/* The reference's speculative output head for greedy decoding
 * (src/archs/transformer/forward/spec_head.c), over a tied F16 table in device memory: an int8
 * sketch of the table ranks the vocabulary, only the best-ranked rows get their exact logit.
 *
 * geist_hip_spec_head_geometry: the sizes spec_head_build would choose (spec_head.c:431-452):
 * sketch width d_model / stride, stride = d_model / 640 lowered until it divides d_model
 * (stride_override > 0 as GEIST_SPEC_STRIDE), finalists 1024 or, from 200000 tokens on, 4096
 * (topk_override > 0 as GEIST_SPEC_TOPK, clamped to 16..n_vocab). GEIST_HIP_E_UNSUPPORTED where
 * the reference builds no sketch (n_vocab < 8192, or a sketch row not 3x smaller than a table
 * row) and where this implementation does not: sketch width not a multiple of 16 or above 1040,
 * d_model not a multiple of 8 or above 5120, more finalists than n_vocab / 64 (the finalists
 * are found among the rows that reach the topk-th largest maximum of groups of 32 scores; with
 * at most every second group involved that is about 1.4 x topk rows).
 *
 * geist_hip_spec_head_build replaces spec_head_build (spec_head.c:402-607), run once per model:
 * the sketch_dim dimensions of largest variance over every (n_vocab / 512)-th row, each row's
 * values there as int8 with one scale per row, and the two row norms of the certainty bound.
 * Kept dimensions, int8 values and scales equal the reference's as written (strict IEEE
 * evaluation); the norms agree to rounding. d_embed_f16 must stay valid while the head is used.
 *
 * geist_hip_spec_head_try replaces transformer_spec_head_try (spec_head.c:624-889) for one
 * normed hidden row: rough scores over the sketch, the topk best of them, exact logits of those
 * rows in the arithmetic of f16_gemv_m1, the best of them (lowest index first). *d_result
 * (device memory) receives the token and answered = 1, or answered = 0 when the head declines
 * and the caller has to run the dense head: with verify != 0 (GEIST_SPEC_VERIFY=1) whenever an
 * excluded row's upper bound reaches the winner (spec_head.c:846-872); without it only if more
 * than 2 x topk rows reach the topk-th largest maximum of groups of 32 scores (rough scores
 * that tie in their thousands), which the reference's
 * heap would resolve by its insertion order. Greedy only, as in the reference (spec_head.c:645).
 * Calls that overlap on one head race: it owns the buffers of a call. */
typedef struct geist_hip_spec_head geist_hip_spec_head;
struct geist_hip_spec_result {
    int32_t token;       /* -1 when not answered without verification */
    int32_t answered;
    int32_t n_finalists; /* rows scored exactly: the topk best rough scores */
    int32_t n_listed;    /* candidate rows the finalists were chosen from */
    float   cutoff;      /* the smallest rough score among the finalists */
    float   best_exact;  /* the winner's logit */
};
/* Device pointers into a built head, for inspection. */
struct geist_hip_spec_head_view {
    size_t          n_vocab, d_model, sketch_dim, topk;
    const uint32_t *d_dims;      /* [sketch_dim] ascending */
    const int8_t   *d_sketch;    /* [n_vocab, sketch_dim] */
    const float    *d_row_scale; /* [n_vocab] */
    const float    *d_w_drop;    /* [n_vocab] */
    const float    *d_w_l1;      /* [n_vocab] */
    const float    *d_rough;     /* [n_vocab] rough scores of the last try */
};
int geist_hip_spec_head_geometry(size_t n_vocab, size_t d_model, size_t stride_override,
                                 size_t topk_override, size_t *sketch_dim, size_t *topk);
int geist_hip_spec_head_build(geist_hip_sampler *s, const uint16_t *d_embed_f16, size_t n_vocab,
                              size_t d_model, size_t stride_override, size_t topk_override,
                              geist_hip_spec_head **out);
void geist_hip_spec_head_destroy(geist_hip_sampler *s, geist_hip_spec_head *sh);
int  geist_hip_spec_head_view(const geist_hip_spec_head *sh, struct geist_hip_spec_head_view *out);
int  geist_hip_spec_head_try(geist_hip_sampler *s, geist_hip_spec_head *sh,
                             const float *d_hidden_normed, int verify,
                             struct geist_hip_spec_result *d_result);

/* geist_hip_spec_head_try with the output norm of head.c:99-101 in front, in the same launch as
 * the activation's quantisation: d_hidden is the row before the norm, d_normed [d_model]
 * receives geist_hip_rmsnorm_rows' result for it (bit for bit) and is what the finalists are
 * scored against. */
int geist_hip_spec_head_try_hidden(geist_hip_sampler *s, geist_hip_spec_head *sh,
                                   const float *d_hidden, const float *d_norm_weight,
                                   float rms_eps, float *d_normed, int verify,
                                   struct geist_hip_spec_result *d_result);

#ifdef __cplusplus
}
#endif
#endif
