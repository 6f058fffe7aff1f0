/* Launchers of the output-head kernels (lm_head.hip): the RMS norm in front of the lm_head and
 * the F16 lm_head projection itself, so that logits are born in device memory and the sampler
 * reads them there. */
#ifndef GEIST_LM_HEAD_KERNELS_H
#define GEIST_LM_HEAD_KERNELS_H

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace gs {

constexpr int GEMV_M_MAX = 8; /* activation rows one pass over the weights serves */
constexpr int F64_M_MAX  = 16; /* ... in the double-accumulation projection (a matrix-core tile) */

/* y = x * w * rsqrt(mean(x^2) + eps) per row; y may alias x. */
void launch_rmsnorm_rows(hipStream_t stream, const float *x, long ld_x, const float *w, float eps,
                         int n_rows, int n, float *y, long ld_y);

/* What the projection can do on its way, for n_m <= 2 activation rows (f16_gemv_can_fuse):
 * with tmax != NULL the work is dealt out in the layout of the sampler's top-k scan (chunks of
 * 8192 logits, 256 threads) and tmax[(m * n_chunks + chunk) * 256 + t] receives the maximum of
 * scanning thread t's logits of row m, so that the sampler can skip its own pass over the
 * logits. (Folding the RMS norm into the projection as well was tried: the registers it takes
 * cost the projection more than the small kernel it saves.) */
struct GemvFuse {
    float *tmax;
    int    n_chunks;
    /* Independent of tmax, for one activation row in the plain layout: gmax[g] receives the
     * maximum of the results of the rows 32 g .. 32 g + 31 (the rows one wavefront computes). */
    float *gmax;
};
bool f16_gemv_can_fuse(int n_m);

/* y[m][r] = sum_i f16(W[r][i]) * x[m][i] for m < n_m <= GEMV_M_MAX; n_in a multiple of 8. */
void launch_f16_gemv(hipStream_t stream, const uint16_t *w_f16, long n_out, int n_in,
                     const float *x, long ld_x, int n_m, float *y, long ld_y,
                     const GemvFuse *fuse = nullptr);

/* Scratch of the double-accumulation projection, for one pass of up to F64_M_MAX rows. */
struct F64Scratch {
    double *xd;        /* [F64_M_MAX][n_in] the activations in double */
    double *xs;        /* [F64_M_MAX][ceil(n_in / 64)] their norms per stage of 64 columns */
    int    *amb_count; /* outputs whose rounding depends on the order of the sum ... */
    int2   *amb_list;  /* ... [n_out * F64_M_MAX] (weight row, activation row) */
};
/* The portable kernel (cpu_scalar_w_quant_mN for F16): y[m][r] = (float) sum_i (double) x[m][i] *
 * (double) f16(W[r][i]), the sum as if in index order; n_m <= F64_M_MAX, n_in a multiple of 8. */
void launch_f16_linear_f64(hipStream_t stream, const uint16_t *w_f16, long n_out, int n_in,
                           const float *x, long ld_x, int n_m, const F64Scratch &ws, float *y,
                           long ld_y);

/* Scratch of the Q6_K projection, for one pass of up to Q6K_M_MAX rows. */
constexpr int Q6K_M_MAX = 4;
struct Q6KScratch {
    double *xd;        /* [Q6K_M_MAX][n_in] the activations in double */
    double *xsum;      /* [Q6K_M_MAX][n_in / 16] their sums per group of 16 */
    double *xabs;      /* [Q6K_M_MAX][n_in / 16] the sums of their magnitudes */
    int    *amb_count; /* outputs whose rounding depends on the order of the sum ... */
    int2   *amb_list;  /* ... [n_out * Q6K_M_MAX] (table row, activation row) */
    uint32_t *act8;    /* activations as int8 for the x86 kernels: one row of [n_in / 256][Q8K_ACT_DWORDS]
                        * (Q6_K) or Q4X_M_MAX rows of q4k_x86_act_dwords (Q4_K) */
};
/* One super-block of int8 activations: 64 dwords of four int8 each in element order, sixteen
 * int32 sums per group of sixteen, the scale d_a (binary32 bits), padding. */
constexpr int Q8K_ACT_DWORDS = 96;
/* The portable kernel over a Q6_K table (cpu_scalar_w_quant_m1 / _mN after dequant_q6_K_row):
 * y[m][r] = (float) sum_k (double) x[m][k] * (double) w[r][k], the sum as if in index order;
 * n_m <= Q6K_M_MAX, n_in a multiple of 256, the table 4-byte aligned. */
void launch_q6k_linear(hipStream_t stream, const uint8_t *w_q6k, long n_out, int n_in,
                       const float *x, long ld_x, int n_m, const Q6KScratch &ws, float *y,
                       long ld_y);

/* The Q6_K table in the order the device reads it (lm_head_q6k.hip): bytes of the packed copy,
 * the packing kernel (once per model), and the projection over the packed copy, which adds in
 * the reference's order and needs no second kernel. */
size_t q6k_packed_bytes(long n_out, int n_in);
void launch_q6k_pack(hipStream_t stream, const uint8_t *w_q6k, long n_out, int n_in, void *packed);
void launch_q6k_packed_linear(hipStream_t stream, const void *packed, long n_out, int n_in,
                              const float *x, long ld_x, int n_m, const Q6KScratch &ws, float *y,
                              long ld_y);
/* The x86 backend's decode kernel (q6k_gemv_m1, src/backends/cpu_x86/kernel_q6k_gemv.c) over the
 * packed copy (lm_head_q6k_x86.hip), in its two parts: the activations of n_m rows as int8 per
 * super-block (act: [n_m][n_in / 256][Q8K_ACT_DWORDS]), and one row's integer dot products with
 * binary32 accumulation in the reference's order. launch_rmsnorm_q8k_rows is launch_rmsnorm_rows
 * and the quantiser in one launch (n a multiple of 256). */
void launch_q8k_quantize(hipStream_t stream, const float *x, long ld_x, int n_m, int n_in,
                         uint32_t *act);
void launch_rmsnorm_q8k_rows(hipStream_t stream, const float *x, long ld_x, const float *w,
                             float eps, int n_rows, int n, float *y, long ld_y, uint32_t *act);
void launch_q6k_packed_gemv_q8k(hipStream_t stream, const void *packed, long n_out, int n_in,
                                const uint32_t *act, float *y);
/* ... and over the table as it lies in the file (4-byte aligned). */
void launch_q6k_gemv_q8k(hipStream_t stream, const uint8_t *w_q6k, long n_out, int n_in,
                         const uint32_t *act, float *y);
/* The x86 backend's batch path over a Q6_K table (cpu_x86_linear_q6k_mN,
 * src/backends/cpu_x86/linear_q6k.c:234-300) over the packed copy or the table as it lies: the rows as int8 with one scale
 * each (quantize_x_int8_sym; act: per row q6k_x86_batch_act_dwords(n_in) dwords), and the integer
 * dot products per group of sixteen of n_m <= Q6X_M_MAX rows in one pass over the table, joined
 * in binary32 as the W8A8 lane kernels of a VNNI host join them (lanes) or as the scalar kernel
 * does. */
constexpr int Q6X_M_MAX = 8;
size_t q6k_x86_batch_act_dwords(int n_in);
void launch_q8s_row_quantize(hipStream_t stream, const float *x, long ld_x, int n_m, int n_in,
                             uint32_t *act);
void launch_rmsnorm_q8s_rows(hipStream_t stream, const float *x, long ld_x, const float *w,
                             float eps, int n_rows, int n, float *y, long ld_y, uint32_t *act);
/* table: the packed copy (packed) or the table as it lies in the file (4-byte aligned) */
void launch_q6k_gemm_q8s(hipStream_t stream, const void *table, bool packed, long n_out, int n_in,
                         const uint32_t *act, int n_m, bool lanes, float *y, long ld_y);
/* The x86 backend's kernels over a Q4_K table -- the decode kernel q4kx8_gemv_m1
 * (src/backends/cpu_x86/kernel_q4kx8_gemm_avx512.c) and the batch path of
 * cpu_x86_linear_q4k_mN (linear_q4k.c:198-250) -- over the packed copy (lm_head_q4k_x86.hip):
 * the activations of n_m rows as int8 with one scale per row (act: per row
 * q4k_x86_act_dwords(n_in) dwords; ties_even: the batch quantiser quantize_q8_Kx4 instead of the
 * decode kernel's), and the integer dot products of n_m <= Q4X_M_MAX rows in one pass over the
 * table, with binary32 accumulation in the reference's order (pairs: that of its 16 x 16
 * AVX-512 tiles, once per pair of sub-blocks). */
constexpr int Q4X_ACT_DWORDS = 72; /* 64 of int8 (even / odd elements of every eight), 8 sums */
constexpr int Q4X_ACT_TAIL   = 8;  /* the row's scale, and padding to 32 bytes */
constexpr int Q4X_M_MAX      = 8;
size_t q4k_x86_act_dwords(int n_in);
void launch_q8k_row_quantize(hipStream_t stream, const float *x, long ld_x, int n_m, int n_in,
                             bool ties_even, uint32_t *act);
/* launch_rmsnorm_rows and that quantiser in one launch (n a multiple of 256) */
void launch_rmsnorm_q8k_row_rows(hipStream_t stream, const float *x, long ld_x, const float *w,
                                 float eps, int n_rows, int n, float *y, long ld_y, bool ties_even,
                                 uint32_t *act);
void launch_q4k_packed_gemv_q8k(hipStream_t stream, const void *packed, long n_out, int n_in,
                                const uint32_t *act, int n_m, bool pairs, float *y, long ld_y);
/* The same for a Q4_K table (packed form only; 148 bytes per block of 144): n_in a multiple of
 * 256, the table 4-byte aligned. The scratch is the Q6_K projection's. */
size_t q4k_packed_bytes(long n_out, int n_in);
void launch_q4k_pack(hipStream_t stream, const uint8_t *w_q4k, long n_out, int n_in, void *packed);
void launch_q4k_packed_linear(hipStream_t stream, const void *packed, long n_out, int n_in,
                              const float *x, long ld_x, int n_m, const Q6KScratch &ws, float *y,
                              long ld_y);

/* The same for the int8 form of the table (q8w_gemv_m1): y[m][r] = (sum_i wq[r][i] * x[m][i]) *
 * scales[r]; n_in a multiple of 16. */
void launch_q8w_gemv(hipStream_t stream, const int8_t *wq, const float *scales, long n_out,
                     int n_in, const float *x, long ld_x, int n_m, float *y, long ld_y,
                     const GemvFuse *fuse = nullptr);
/* f16_to_q8w: wq [n_out][n_in] and scales [n_out] from the binary16 table. */
void launch_f16_to_q8w(hipStream_t stream, const uint16_t *w_f16, long n_out, int n_in, int8_t *wq,
                       float *scales);

} // namespace gs
#endif
