/*
 * lm_head_q4k_x86.hip -- the lm_head projection of one activation row over a Q4_K table with the
 * results of the reference's x86 decode kernel q4kx8_gemv_m1
 * (src/backends/cpu_x86/kernel_q4kx8_gemm_avx512.c:47-77 the activation quantiser, :81-304 the dot
 * products of one row against eight interleaved table rows, :380-399 the sweep; reached from
 * cpu_x86_linear_q4k_m1, src/backends/cpu_x86/linear_q4k.c:163-166, for tables of a multiple of
 * 8 rows). The reference interleaves eight table rows so that eight outputs fill the lanes of a
 * vector; each output's arithmetic involves its own row alone:
 *   activations  ONE scale for the row: amax = max |x|, d_a = amax / 127 (1 when amax is 0),
 *                a = (int) (x / d_a +- 0.5) (round half away from zero), clamped to int8;
 *   per block    integers: I = sum over the eight sub-blocks j of 32 of scale_j * (sum q * a),
 *                M = sum_j min_j * (sum of a over sub-block j); binary32:
 *                acc = fmaf((float) I, d * d_a, acc), acc_min = fmaf((float) M, dmin * d_a,
 *                acc_min), the two products rounded to binary32 first;
 *   result       y = acc - acc_min.
 * The integers cannot overflow (|I| < 2^26), so their order is free; the binary32 steps are the
 * reference's, which makes the result the reference's bit for bit. Finite activations only.
 *
 * The table is read from the packed copy of geist_hip_q4k_pack (lm_head_q6k.hip): a lane owns a
 * table row; a dword holds the 4-bit values of eight consecutive elements, one mask gives the
 * even ones as bytes and a shift and a mask the odd ones, and two v_dot4_i32_i8 multiply them
 * with the activations, which the quantiser lays out to match (per eight elements a dword of the
 * even ones and a dword of the odd ones) and which are scalar operands.
 */
#include "lm_head_kernels.h"
#include "rmsnorm_device.h"

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gs {

constexpr int Q4X_TPB         = 256;
constexpr int Q4X_ROW_DWORDS  = 37;
constexpr int Q4X_PACK_DWORDS = Q4X_ROW_DWORDS * 64; /* the packed copy's dwords per (64 rows, block) */

/* Thread t's element of a super-block, given the reciprocal of the row's scale: its int8 value
 * into the block's dwords (ob), the sums per sub-block of 32 behind them. */
__device__ __forceinline__ void q4x_quantize_block(float xv, float inv, bool ties_even,
                                                   uint32_t *__restrict__ ob) {
    const int   t = threadIdx.x;
    const float v = __fmul_rn(xv, inv);
    /* the decode kernel's quantiser rounds half away from zero by truncation and clamps; the
     * batch quantiser is lrintf (|v| <= 127 up to rounding: nothing to clamp) */
    int q = ties_even ? __float2int_rn(v)
                      : __float2int_rz(v < 0.0f ? __fsub_rn(v, 0.5f) : __fadd_rn(v, 0.5f));
    q     = q < -128 ? -128 : q > 127 ? 127 : q;
    int sum       = q;
#pragma unroll
    for (int s = 16; s >= 1; s >>= 1)
        sum += __shfl_xor(sum, s);
    const uint32_t b0 = (uint32_t) q & 0xffu;
    const uint32_t b1 = (uint32_t) __shfl_down(q, 2) & 0xffu;
    const uint32_t b2 = (uint32_t) __shfl_down(q, 4) & 0xffu;
    const uint32_t b3 = (uint32_t) __shfl_down(q, 6) & 0xffu;
    if ((t & 7) < 2) /* elements 8 k + {0, 2, 4, 6} to dword 2 k, 8 k + {1, 3, 5, 7} to 2 k + 1 */
        ob[2 * (t >> 3) + (t & 7)] = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
    if ((t & 31) == 0)
        ob[64 + (t >> 5)] = (uint32_t) sum;
}

/* One workgroup per activation row. act: per row q4k_x86_act_dwords dwords: per super-block
 * Q4X_ACT_DWORDS -- 64 of int8 (per eight elements the even ones, then the odd ones), eight
 * int32 sums per sub-block of 32 --, and behind the row's last block the scale d_a as binary32
 * (and padding that keeps the next row 32-byte aligned). ties_even: the batch quantiser
 * (quantize_q8_Kx4, q8_kx4.c:21-105) instead of the decode kernel's. */
__global__ __launch_bounds__(Q4X_TPB) void k_q8k_row_quantize(const float *__restrict__ x, long ld_x,
                                                             int nb, bool ties_even,
                                                             uint32_t *__restrict__ act) {
    __shared__ float s_max[Q4X_TPB / 64];
    const int        m = blockIdx.x, t = threadIdx.x;
    const float     *xr = x + (long) m * ld_x;
    uint32_t        *o  = act + (long) m * ((long) nb * Q4X_ACT_DWORDS + Q4X_ACT_TAIL);
    float            ax = 0.0f;
    for (int b = 0; b < nb; ++b)
        ax = __builtin_fmaxf(ax, __builtin_fabsf(xr[256 * b + t])); /* (a NaN is passed over) */
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1)
        ax = __builtin_fmaxf(ax, __shfl_xor(ax, s));
    if ((t & 63) == 0)
        s_max[t >> 6] = ax;
    __syncthreads();
    const float amax  = __builtin_fmaxf(__builtin_fmaxf(s_max[0], s_max[1]),
                                        __builtin_fmaxf(s_max[2], s_max[3]));
    const float scale = amax == 0.0f ? 1.0f : __fdiv_rn(amax, 127.0f);
    const float inv   = __fdiv_rn(1.0f, scale);
    if (t == 0)
        o[(long) nb * Q4X_ACT_DWORDS] = __float_as_uint(scale);
    for (int b = 0; b < nb; ++b)
        q4x_quantize_block(xr[256 * b + t], inv, ties_even, o + (long) b * Q4X_ACT_DWORDS);
}

/* The output norm (cpu_scalar_rmsnorm, as k_rmsnorm_rows computes it) and that quantiser in one
 * launch, one workgroup per row: the normed row goes to y and, as int8, to act. A thread reads
 * back what it wrote itself. n a multiple of 256. */
__global__ __launch_bounds__(Q4X_TPB) void k_rmsnorm_q8k_row_rows(const float *__restrict__ x,
                                                                 long ld_x,
                                                                 const float *__restrict__ w,
                                                                 float eps, int n,
                                                                 float *__restrict__ y, long ld_y,
                                                                 bool ties_even,
                                                                 uint32_t *__restrict__ act) {
    __shared__ double s_part[Q4X_TPB];
    __shared__ float  s_inv;
    __shared__ float  s_max[Q4X_TPB / 64];
    const int    nb = n / 256, m = blockIdx.x, t = threadIdx.x;
    const float *xr = x + (long) m * ld_x;
    float       *yr = y + (long) m * ld_y;
    uint32_t    *o  = act + (long) m * ((long) nb * Q4X_ACT_DWORDS + Q4X_ACT_TAIL);
    const float  rinv = block_rms_inv<Q4X_TPB>(xr, n, eps, s_part, &s_inv);
    float        ax = 0.0f;
    for (int b = 0; b < nb; ++b) {
        const int   i = 256 * b + t;
        const float v = __fmul_rn(__fmul_rn(xr[i], rinv), w[i]);
        yr[i]         = v;
        ax            = __builtin_fmaxf(ax, __builtin_fabsf(v));
    }
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1)
        ax = __builtin_fmaxf(ax, __shfl_xor(ax, s));
    if ((t & 63) == 0)
        s_max[t >> 6] = ax;
    __syncthreads();
    const float amax  = __builtin_fmaxf(__builtin_fmaxf(s_max[0], s_max[1]),
                                        __builtin_fmaxf(s_max[2], s_max[3]));
    const float scale = amax == 0.0f ? 1.0f : __fdiv_rn(amax, 127.0f);
    const float inv   = __fdiv_rn(1.0f, scale);
    if (t == 0)
        o[(long) nb * Q4X_ACT_DWORDS] = __float_as_uint(scale);
    for (int b = 0; b < nb; ++b)
        q4x_quantize_block(yr[256 * b + t], inv, ties_even, o + (long) b * Q4X_ACT_DWORDS);
}

typedef uint32_t q4x_u4 __attribute__((ext_vector_type(4)));

struct Q4xBlock {
    uint32_t q[32]; /* the 4-bit values, eight consecutive elements to a dword */
    uint32_t sc[2]; /* the eight scales as bytes */
    uint32_t mn[2]; /* the eight minima as bytes */
    uint32_t dd;    /* d (low half) and dmin, binary16 */
};
__device__ __forceinline__ void q4x_load(const uint32_t *__restrict__ base, int r, Q4xBlock &k) {
#pragma unroll
    for (int p = 0; p < 8; ++p) {
        const q4x_u4 t =
            __builtin_nontemporal_load(reinterpret_cast<const q4x_u4 *>(base + p * 256 + 4 * r));
        k.q[4 * p] = t.x, k.q[4 * p + 1] = t.y, k.q[4 * p + 2] = t.z, k.q[4 * p + 3] = t.w;
    }
    const q4x_u4 t =
        __builtin_nontemporal_load(reinterpret_cast<const q4x_u4 *>(base + 8 * 256 + 4 * r));
    k.sc[0] = t.x, k.sc[1] = t.y, k.mn[0] = t.z, k.mn[1] = t.w;
    k.dd    = __builtin_nontemporal_load(base + 2304 + r);
}

/* M activation rows share a pass over the table. PAIRS: the binary32 accumulators are joined once
 * per pair of sub-blocks (the reference's 16 x 16 AVX-512 tiles,
 * kernel_q4kx8_gemm_avx512_full.c:94, 729-778) instead of once per super-block. */
template <int M, bool PAIRS>
__global__ __launch_bounds__(Q4X_TPB, PAIRS && M > 2 ? 3 : 4) void k_q4k_packed_gemv_x86(
    const uint32_t *__restrict__ packed, long n_out, int nb, const uint32_t *__restrict__ act,
    float *__restrict__ y, long ld_y) {
    const int  r = threadIdx.x & 63;
    const long g = (long) blockIdx.x * (Q4X_TPB / 64) + threadIdx.x / 64;
    if (g * 64 >= n_out)
        return;
    const long      row    = g * 64 + r;
    const uint32_t *base   = packed + g * nb * Q4X_PACK_DWORDS;
    const long      act_ld = (long) nb * Q4X_ACT_DWORDS + Q4X_ACT_TAIL;
    float           d_a[M], acc[M], acc_min[M];
#pragma unroll
    for (int m = 0; m < M; ++m) {
        d_a[m] = __uint_as_float(act[m * act_ld + (long) nb * Q4X_ACT_DWORDS]);
        acc[m] = 0.0f, acc_min[m] = 0.0f;
    }
    /* a block ahead: the next block's loads are in flight while this one is worked on */
    Q4xBlock cur, nxt;
    q4x_load(base, r, cur);
    for (int b = 0; b < nb; ++b) {
        if (b + 1 < nb)
            q4x_load(base + (long) (b + 1) * Q4X_PACK_DWORDS, r, nxt);
        const uint32_t *a = act + (long) b * Q4X_ACT_DWORDS; /* uniform: scalar loads */
        typedef uint32_t u8v __attribute__((ext_vector_type(8)));
        const float d    = __half2float(__ushort_as_half((unsigned short) (cur.dd & 0xffffu)));
        const float dmin = __half2float(__ushort_as_half((unsigned short) (cur.dd >> 16)));
        int         iacc[M];
#pragma unroll
        for (int m = 0; m < M; ++m)
            iacc[m] = 0;
        /* With several rows the scalar loads stay near their arithmetic, four rows at a time:
         * a fence that loads may not pass and that needs the sums so far. Hoisted to the top of
         * the block they would not fit the scalar registers. */
        /* the minima against the activations' sums per sub-block: a chain of its own */
#pragma unroll
        for (int m = 0; m < M; ++m) {
            if (M > 4 && m % 4 == 0)
                asm volatile("" : "+v"(acc_min[m > 0 ? m - 1 : 0])::"memory");
            const u8v   bs = *reinterpret_cast<const u8v *>(a + m * act_ld + 64);
            const float dm = __fmul_rn(dmin, d_a[m]);
            int         im = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                im += __mul24((int) ((cur.mn[j >> 2] >> (8 * (j & 3))) & 0xffu), (int) bs[j]);
                if (PAIRS ? (j & 1) : j == 7) {
                    acc_min[m] = __builtin_fmaf((float) im, dm, acc_min[m]);
                    im         = 0;
                }
            }
        }
        /* Steps of (sub-block j, group of up to four rows). The activations of a step are
         * scalar loads issued one step ahead, before the fence that opens the step. */
        constexpr int G  = M < 4 ? M : 4;
        constexpr int NG = (M + G - 1) / G;
        u8v           avc[G], avn[G];
        uint32_t      even[4], odd[4];
        int           sc = 0;
        if (M > 1) {
#pragma unroll
            for (int i = 0; i < G; ++i)
                avc[i] = *reinterpret_cast<const u8v *>(a + i * act_ld);
        }
#pragma unroll
        for (int st = 0; st < 8 * NG; ++st) {
            const int j = st / NG, grp = st % NG; /* sub-block j: elements 32 j .. 32 j + 31 */
            if (M > 1) {
                if (st + 1 < 8 * NG) {
                    const int jn = (st + 1) / NG, gn = (st + 1) % NG;
#pragma unroll
                    for (int i = 0; i < G; ++i)
                        if (gn * G + i < M)
                            avn[i] = *reinterpret_cast<const u8v *>(a + (gn * G + i) * act_ld + 8 * jn);
                }
#pragma unroll
                for (int i = 0; i < M; ++i)
                    asm volatile("" : "+v"(iacc[i])::"memory");
            }
            if (grp == 0) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t w = cur.q[4 * j + k];
                    even[k] = w & 0x0f0f0f0fu, odd[k] = (w >> 4) & 0x0f0f0f0fu;
                }
                sc = (int) ((cur.sc[j >> 2] >> (8 * (j & 3))) & 0xffu);
            }
#pragma unroll
            for (int i = 0; i < G; ++i) {
                const int m = grp * G + i;
                if (m >= M)
                    continue;
                const u8v av  = M > 1 ? avc[i] : *reinterpret_cast<const u8v *>(a + 8 * j);
                int       dot = 0;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    dot = __builtin_amdgcn_sdot4((int) even[k], (int) av[2 * k], dot, false);
                    dot = __builtin_amdgcn_sdot4((int) odd[k], (int) av[2 * k + 1], dot, false);
                }
                iacc[m] += __mul24(sc, dot);
                if (PAIRS && (j & 1)) {
                    acc[m]  = __builtin_fmaf((float) iacc[m], __fmul_rn(d, d_a[m]), acc[m]);
                    iacc[m] = 0;
                }
            }
            if (M > 1) {
#pragma unroll
                for (int i = 0; i < G; ++i)
                    avc[i] = avn[i];
            }
        }
        if (!PAIRS) {
#pragma unroll
            for (int m = 0; m < M; ++m)
                acc[m] = __builtin_fmaf((float) iacc[m], __fmul_rn(d, d_a[m]), acc[m]);
        }
        if (b + 1 < nb)
            cur = nxt;
    }
    if (row < n_out) {
#pragma unroll
        for (int m = 0; m < M; ++m)
            y[m * ld_y + row] = __fsub_rn(acc[m], acc_min[m]);
    }
}

size_t q4k_x86_act_dwords(int n_in) {
    return (size_t) (n_in / 256) * Q4X_ACT_DWORDS + Q4X_ACT_TAIL;
}

void launch_q8k_row_quantize(hipStream_t stream, const float *x, long ld_x, int n_m, int n_in,
                             bool ties_even, uint32_t *act) {
    k_q8k_row_quantize<<<dim3(n_m), dim3(Q4X_TPB), 0, stream>>>(x, ld_x, n_in / 256, ties_even, act);
}

void launch_rmsnorm_q8k_row_rows(hipStream_t stream, const float *x, long ld_x, const float *w,
                                 float eps, int n_rows, int n, float *y, long ld_y, bool ties_even,
                                 uint32_t *act) {
    k_rmsnorm_q8k_row_rows<<<dim3(n_rows), dim3(Q4X_TPB), 0, stream>>>(x, ld_x, w, eps, n, y, ld_y,
                                                                      ties_even, act);
}

template <int M>
static void q4x_launch(hipStream_t stream, const uint32_t *packed, long n_out, int nb,
                       const uint32_t *act, bool pairs, float *y, long ld_y) {
    const long groups = (n_out + 63) / 64;
    const dim3 grid((unsigned) ((groups + 3) / 4)), block(Q4X_TPB);
    if (pairs)
        k_q4k_packed_gemv_x86<M, true><<<grid, block, 0, stream>>>(packed, n_out, nb, act, y, ld_y);
    else
        k_q4k_packed_gemv_x86<M, false><<<grid, block, 0, stream>>>(packed, n_out, nb, act, y, ld_y);
}

void launch_q4k_packed_gemv_q8k(hipStream_t stream, const void *packed, long n_out, int n_in,
                                const uint32_t *act, int n_m, bool pairs, float *y, long ld_y) {
    const uint32_t *p  = static_cast<const uint32_t *>(packed);
    const int       nb = n_in / 256;
    switch (n_m) {
    case 1: q4x_launch<1>(stream, p, n_out, nb, act, pairs, y, ld_y); break;
    case 2: q4x_launch<2>(stream, p, n_out, nb, act, pairs, y, ld_y); break;
    case 3: q4x_launch<3>(stream, p, n_out, nb, act, pairs, y, ld_y); break;
    case 4: q4x_launch<4>(stream, p, n_out, nb, act, pairs, y, ld_y); break;
    case 5: q4x_launch<5>(stream, p, n_out, nb, act, pairs, y, ld_y); break;
    case 6: q4x_launch<6>(stream, p, n_out, nb, act, pairs, y, ld_y); break;
    case 7: q4x_launch<7>(stream, p, n_out, nb, act, pairs, y, ld_y); break;
    default: q4x_launch<8>(stream, p, n_out, nb, act, pairs, y, ld_y); break;
    }
}

} // namespace gs
