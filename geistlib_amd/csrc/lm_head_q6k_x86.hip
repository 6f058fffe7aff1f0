/*
 * lm_head_q6k_x86.hip -- the lm_head projection of one activation row over a Q6_K table with the
 * results of the reference's x86 decode kernel q6k_gemv_m1
 * (src/backends/cpu_x86/kernel_q6k_gemv.c:43-67 the activation quantiser, :90-157 the dot
 * product, called from cpu_x86_linear_q6k_m1, src/backends/cpu_x86/linear_q6k.c:205-207).
 *
 * Arithmetic of the reference, per super-block of 256 elements:
 *   activations  amax = max |x|, d_a = amax / 127, a = lrintf(x * (127 / amax)) as int8 (all zero
 *                when amax is zero), s[g] = sum of a over group g of sixteen;
 *   weights      q in 0..63 (six bits), a scale per sixteen elements (int8), d_w (binary16);
 *   integers     eight lanes: lane u adds, over the eight runs v of 32 elements, scale[2 v +
 *                (u >> 2)] * (the four products q * a of elements 32 v + 4 u .. + 3), and loses
 *                32 * (s[2 u] scale[2 u] + s[2 u + 1] scale[2 u + 1]);
 *   binary32     acc[u] = fmaf(d_a * d_w, (float) lane[u], acc[u]); after the last block
 *                y = ((acc0 + acc4) + (acc1 + acc5)) + ((acc2 + acc6) + (acc3 + acc7)).
 * The integer part cannot overflow (|lane| < 2^26), so its order is free; the binary32 part is
 * done here in the reference's order, which makes the result the reference's bit for bit.
 * Activations are taken to be finite (a NaN or an infinity sends lrintf out of int8's range,
 * where the reference's own result is whatever the conversion leaves).
 *
 * The table is read from the packed copy of geist_hip_q6k_pack (lm_head_q6k.hip): a lane owns a
 * table row and gets a block as thirteen 16-byte pieces and one dword, the six-bit values in
 * element order. The four values of one integer dot product are 24 consecutive bits; five
 * bit-field instructions spread them over the four bytes of a dword, v_dot4_i32_i8 multiplies
 * them with four int8 activations (a scalar operand: the activations are uniform over the
 * wavefront), and v_mad_i32_i24 applies the scale.
 */
#include "lm_head_kernels.h"
#include "lm_head_q6k_block.h"
#include "rmsnorm_device.h"

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gs {

constexpr int Q6X_TPB         = 256;
constexpr int Q6X_PACK_DWORDS = 53 * 64; /* the packed copy's dwords per (64 rows, block) */

/* One super-block's 256 activations, one to a thread of the workgroup, as int8 (64 dwords, four
 * to a dword in element order), their sixteen sums per group of sixteen as int32, and d_a, written
 * to o[0 .. Q8K_ACT_DWORDS). s_max: four floats that no thread still reads from an earlier call
 * (the callers alternate between two). */
__device__ __forceinline__ void q8k_quantize_block(float xv, uint32_t *__restrict__ o,
                                                   float *s_max) {
    const int t  = threadIdx.x;
    float     ax = __builtin_fabsf(xv);
    /* the reference keeps the running maximum when a comparison with a NaN fails; fmaxf drops
     * the NaN in the same way */
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1)
        ax = __builtin_fmaxf(ax, __shfl_xor(ax, s));
    if ((t & 63) == 0)
        s_max[t >> 6] = ax;
    __syncthreads();
    const float amax = __builtin_fmaxf(__builtin_fmaxf(s_max[0], s_max[1]),
                                       __builtin_fmaxf(s_max[2], s_max[3]));
    const float id   = amax > 0.0f ? __fdiv_rn(127.0f, amax) : 0.0f;
    const int   q    = __float2int_rn(__fmul_rn(xv, id)); /* lrintf: to nearest, ties to even */
    int         sum  = q;
#pragma unroll
    for (int s = 8; s >= 1; s >>= 1)
        sum += __shfl_xor(sum, s);
    const uint32_t b0 = (uint32_t) q & 0xffu;
    const uint32_t b1 = (uint32_t) __shfl_down(q, 1) & 0xffu;
    const uint32_t b2 = (uint32_t) __shfl_down(q, 2) & 0xffu;
    const uint32_t b3 = (uint32_t) __shfl_down(q, 3) & 0xffu;
    if ((t & 3) == 0)
        o[t >> 2] = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
    if ((t & 15) == 0)
        o[64 + (t >> 4)] = (uint32_t) sum;
    if (t == 0)
        o[80] = __float_as_uint(__fdiv_rn(amax, 127.0f));
}

/* One workgroup per (super-block, activation row). */
__global__ __launch_bounds__(Q6X_TPB) void k_q8k_quantize(const float *__restrict__ x, long ld_x,
                                                         int nb, uint32_t *__restrict__ act) {
    __shared__ float s_max[Q6X_TPB / 64];
    const int        b = blockIdx.x, m = blockIdx.y;
    q8k_quantize_block(x[(long) m * ld_x + (long) b * 256 + threadIdx.x],
                       act + ((long) m * nb + b) * Q8K_ACT_DWORDS, s_max);
}

/* The output norm (cpu_scalar_rmsnorm, src/backends/cpu_scalar/elementwise.c:241-280, as
 * k_rmsnorm_rows computes it) and the quantiser in one launch, one workgroup per row: the normed
 * row goes to y and, as int8 super-blocks, to act. n a multiple of 256. */
__global__ __launch_bounds__(Q6X_TPB) void k_rmsnorm_q8k_rows(const float *__restrict__ x,
                                                             long ld_x,
                                                             const float *__restrict__ w,
                                                             float eps, int n,
                                                             float *__restrict__ y, long ld_y,
                                                             uint32_t *__restrict__ act) {
    __shared__ double s_part[Q6X_TPB];
    __shared__ float  s_inv;
    __shared__ float  s_max[2][Q6X_TPB / 64];
    const int    nb = n / 256, m = blockIdx.x, t = threadIdx.x;
    const float *xr = x + (long) m * ld_x;
    const float  inv = block_rms_inv<Q6X_TPB>(xr, n, eps, s_part, &s_inv);
    for (int b = 0; b < nb; ++b) {
        const int   i = 256 * b + t;
        const float v = __fmul_rn(__fmul_rn(xr[i], inv), w[i]);
        y[(long) m * ld_y + i] = v;
        q8k_quantize_block(v, act + ((long) m * nb + b) * Q8K_ACT_DWORDS, s_max[b & 1]);
    }
}

typedef uint32_t q6x_u4 __attribute__((ext_vector_type(4)));

/* six of a lane's 16-byte pieces of a packed block, from piece p0 on: half a block's values */
__device__ __forceinline__ void q6x_load6(const uint32_t *__restrict__ base, int r, int p0,
                                          uint32_t (&q)[24]) {
#pragma unroll
    for (int p = 0; p < 6; ++p) {
        const q6x_u4 t = __builtin_nontemporal_load(
            reinterpret_cast<const q6x_u4 *>(base + (p0 + p) * 256 + 4 * r));
        q[4 * p] = t.x, q[4 * p + 1] = t.y, q[4 * p + 2] = t.z, q[4 * p + 3] = t.w;
    }
}
__device__ __forceinline__ void q6x_load_scales(const uint32_t *__restrict__ base, int r,
                                                uint32_t (&sc)[4], uint32_t &d52) {
    const q6x_u4 t =
        __builtin_nontemporal_load(reinterpret_cast<const q6x_u4 *>(base + 12 * 256 + 4 * r));
    sc[0] = t.x, sc[1] = t.y, sc[2] = t.z, sc[3] = t.w;
    d52   = __builtin_nontemporal_load(base + 3328 + r);
}
/* scale k of a block (k = 0..15), sign extended */
__device__ __forceinline__ int q6x_scale(const uint32_t (&sc)[4], int k) {
    return __builtin_amdgcn_sbfe((int) sc[k >> 2], 8 * (k & 3), 8);
}
/* The four six-bit values in bits 8 sh .. 8 sh + 23 of the 64 bits hi:lo, one to a byte: twelve
 * bits to each half first (bits 12..15 and 28..31 of y hold strays), then six to each byte. The
 * empty asm keeps the two steps apart: merged, they cost the compiler three instructions more. */
template <int SH>
__device__ __forceinline__ uint32_t q6x_spread(uint32_t lo, uint32_t hi) {
    uint32_t x, t; /* the field from bit 0 on, and the same shifted left by four */
    if (SH == 0)
        x = lo, t = lo << 4;
    else if (SH == 1)
        x = lo >> 8, t = lo >> 4;
    else
        x = __builtin_amdgcn_alignbit(hi, lo, 8 * SH), t = __builtin_amdgcn_alignbit(hi, lo, 8 * SH - 4);
    uint32_t y = (x & 0xfffu) | (t & ~0xfffu);
    asm("" : "+v"(y));
    return ((y << 2) & 0x3f003f00u) | (y & 0x003f003fu);
}
/* The 128 elements of half a block (runs 4 half .. 4 half + 3): lane[u] += scale * (q . a). A
 * run's eight dot products are formed before any of them is used: a dependent instruction right
 * behind a dot product waits. */
__device__ __forceinline__ void q6x_half(const uint32_t (&q)[24], const uint32_t (&sc)[4],
                                         int half, const uint32_t *__restrict__ a,
                                         int (&lane)[8]) {
#pragma unroll
    for (int vl = 0; vl < 4; ++vl) {
        const int v   = 4 * half + vl;
        const int s_a = q6x_scale(sc, 2 * v), s_b = q6x_scale(sc, 2 * v + 1);
        int       dot[8];
        /* the run's 32 activations: one scalar load of eight dwords */
        typedef uint32_t u8v __attribute__((ext_vector_type(8)));
        const u8v av = *reinterpret_cast<const u8v *>(a + 8 * v);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            /* field f of the half: bits 24 f .. 24 f + 23 of its 24 dwords */
            const int      f = 8 * vl + u, w0 = (3 * f) >> 2, sh = (3 * f) & 3;
            const uint32_t lo = q[w0], hi = q[w0 + 1 < 24 ? w0 + 1 : 23];
            const uint32_t z  = sh == 0   ? q6x_spread<0>(lo, hi)
                                : sh == 1 ? q6x_spread<1>(lo, hi)
                                : sh == 2 ? q6x_spread<2>(lo, hi)
                                          : q6x_spread<3>(lo, hi);
            dot[u] = __builtin_amdgcn_sdot4((int) z, (int) av[u], 0, false);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            lane[u] += __mul24(u < 4 ? s_a : s_b, dot[u]);
    }
}

__global__ __launch_bounds__(Q6X_TPB, 4) void k_q6k_packed_gemv_x86(
    const uint32_t *__restrict__ packed, long n_out, int nb, const uint32_t *__restrict__ act,
    float *__restrict__ y) {
    const int  r = threadIdx.x & 63;
    const long g = (long) blockIdx.x * (Q6X_TPB / 64) + threadIdx.x / 64;
    if (g * 64 >= n_out)
        return;
    const long row = g * 64 + r;
    float      acc[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
        acc[u] = 0.0f;
    /* loads run half a block ahead of the arithmetic, as in k_q6k_packed_linear */
    const uint32_t *base = packed + g * nb * Q6X_PACK_DWORDS;
    uint32_t        qa[24], qb[24], sc[4], d52;
    q6x_load_scales(base, r, sc, d52);
    q6x_load6(base, r, 0, qa);
    for (int b = 0; b < nb; ++b) {
        const uint32_t *blk = base + (long) b * Q6X_PACK_DWORDS;
        const uint32_t *a   = act + (long) b * Q8K_ACT_DWORDS; /* uniform: scalar loads */
        q6x_load6(blk, r, 6, qb);
        const float d = __uint_as_float(a[80]) *
                        __half2float(__ushort_as_half((unsigned short) (d52 & 0xffffu)));
        /* the offset of 32 leaves through the activations' sums, paired by scale index */
        typedef uint32_t u16v __attribute__((ext_vector_type(16)));
        const u16v bs = *reinterpret_cast<const u16v *>(a + 64);
        int        lane[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
            lane[u] = -32 * (__mul24((int) bs[2 * u], q6x_scale(sc, 2 * u)) +
                             __mul24((int) bs[2 * u + 1], q6x_scale(sc, 2 * u + 1)));
        uint32_t sc_now[4] = {sc[0], sc[1], sc[2], sc[3]};
        q6x_half(qa, sc_now, 0, a, lane);
        if (b + 1 < nb) {
            q6x_load_scales(blk + Q6X_PACK_DWORDS, r, sc, d52);
            q6x_load6(blk + Q6X_PACK_DWORDS, r, 0, qa);
        }
        q6x_half(qb, sc_now, 1, a, lane);
#pragma unroll
        for (int u = 0; u < 8; ++u)
            acc[u] = __builtin_fmaf(d, (float) lane[u], acc[u]);
    }
    if (row < n_out)
        y[row] = ((acc[0] + acc[4]) + (acc[1] + acc[5])) + ((acc[2] + acc[6]) + (acc[3] + acc[7]));
}

/* The same over the table as it lies in the file, for callers that keep no packed copy: a lane
 * owns a table row and reads its 210-byte blocks whole. There the four low bits and the two high
 * bits of an element lie apart, but in the order the dot product wants them: a dword of ql holds
 * the low nibbles of elements 4u .. 4u + 3 of two runs, a dword of qh the high bits of the same
 * elements of four runs, so a mask and a shift per run put four six-bit values into the bytes of
 * a dword. */
__global__ __launch_bounds__(Q6X_TPB) void k_q6k_gemv_x86(const uint8_t *__restrict__ w,
                                                          long n_out, int nb,
                                                          const uint32_t *__restrict__ act,
                                                          float *__restrict__ y) {
    const long row = (long) blockIdx.x * Q6X_TPB + threadIdx.x;
    if (row >= n_out)
        return;
    const uint8_t *rp = w + row * (long) nb * 210;
    float          acc[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
        acc[u] = 0.0f;
    for (int b = 0; b < nb; ++b) {
        uint32_t d[53];
        q6k_load_block(rp + (long) b * 210, d);
        const uint32_t *a  = act + (long) b * Q8K_ACT_DWORDS; /* uniform: scalar loads */
        const uint32_t  sc[4] = {d[48], d[49], d[50], d[51]};
        const float     dd = __uint_as_float(a[80]) *
                         __half2float(__ushort_as_half((unsigned short) (d[52] & 0xffffu)));
        typedef uint32_t u16v __attribute__((ext_vector_type(16)));
        const u16v bs = *reinterpret_cast<const u16v *>(a + 64);
        int        lane[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
            lane[u] = -32 * (__mul24((int) bs[2 * u], q6x_scale(sc, 2 * u)) +
                             __mul24((int) bs[2 * u + 1], q6x_scale(sc, 2 * u + 1)));
#pragma unroll
        for (int v = 0; v < 8; ++v) { /* run v = 4 h + j: elements 128 h + 32 j .. + 31 */
            const int h = v >> 2, j = v & 3;
            typedef uint32_t u8v __attribute__((ext_vector_type(8)));
            const u8v av  = *reinterpret_cast<const u8v *>(a + 8 * v);
            const int s_a = q6x_scale(sc, 2 * v), s_b = q6x_scale(sc, 2 * v + 1);
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                /* q = nibble (j >> 1) of ql[64 h + 32 (j & 1) + l] | ((qh[32 h + l] >> 2 j) & 3) << 4
                 * for l = 4 u .. 4 u + 3 (src/formats/gguf/q6_K.c:30-36) */
                const uint32_t ql = d[16 * h + 8 * (j & 1) + u], qh = d[32 + 8 * h + u];
                const uint32_t lo = (j >> 1) ? (ql >> 4) & 0x0f0f0f0fu : ql & 0x0f0f0f0fu;
                const uint32_t hi = j == 0   ? (qh << 4) & 0x30303030u
                                    : j == 1 ? (qh << 2) & 0x30303030u
                                    : j == 2 ? qh & 0x30303030u
                                             : (qh >> 2) & 0x30303030u;
                const int dot = __builtin_amdgcn_sdot4((int) (lo | hi), (int) av[u], 0, false);
                lane[u] += __mul24(u < 4 ? s_a : s_b, dot);
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            acc[u] = __builtin_fmaf(dd, (float) lane[u], acc[u]);
    }
    y[row] = ((acc[0] + acc[4]) + (acc[1] + acc[5])) + ((acc[2] + acc[6]) + (acc[3] + acc[7]));
}

/* ---- batches: cpu_x86_linear_q6k_mN (src/backends/cpu_x86/linear_q6k.c:234-300) ---------------
 * The reference multiplies an int8 copy of the table (q6k_to_w8a8_row, q6k_to_w8a8.c:26-68: the
 * six-bit values as bytes, per group of sixteen ws = d * (float) scale and wo = ws * 32) with the
 * rows quantised by quantize_x_int8_sym (src/formats/gguf/common.c:204-250: ONE scale per row,
 * amax / 127, 1 when that is zero; lrintf). Per output and group of sixteen the integer
 * dot = sum of q * a, then in binary32, group after group,
 *   LANES   acc = fmaf(ws, (float) dot, acc); acc = fmaf(-wo, (float) sum_a, acc)   (w8x8_gemm /
 *           w8x16_gemm, kernel_w8a8_avx512_vnni.c:176-297: a host with AVX-512 VNNI, tables of a
 *           multiple of 8 rows)
 *   else    acc = acc + (ws * (float) dot - wo * (float) sum_a), every operation rounded
 *           (w8a8_dot_scalar, kernel_w8a8_scalar.c:14-34, and the VNNI kernel for other tables)
 * and y = scale_x * acc. The device reads the same packed copy as the decode kernel: the values
 * and scales of the int8 copy are in it, and ws is formed as the reference forms it.
 *
 * act, per row (Q8S_ACT_TAIL dwords behind nb blocks of Q8K_ACT_DWORDS): per run of 32 elements
 * twelve dwords -- eight of four int8 each in element order, (float) sum_a of its two groups,
 * -32 * (float) sum_a of the two (exact; fmaf(-wo, s, acc) == fmaf(ws, -32 s, acc) as wo = 32 ws
 * is exact) --, and behind the last block the row's scale. */
constexpr int Q8S_ACT_TAIL = 8;

__device__ __forceinline__ void q8s_quantize_block(float xv, float inv, uint32_t *__restrict__ ob) {
    const int t = threadIdx.x;
    const int q = __float2int_rn(__fmul_rn(xv, inv)); /* lrintf; |x * inv| <= 127 up to rounding */
    int       sum = q;
#pragma unroll
    for (int s = 8; s >= 1; s >>= 1)
        sum += __shfl_xor(sum, s);
    const uint32_t b0 = (uint32_t) q & 0xffu;
    const uint32_t b1 = (uint32_t) __shfl_down(q, 1) & 0xffu;
    const uint32_t b2 = (uint32_t) __shfl_down(q, 2) & 0xffu;
    const uint32_t b3 = (uint32_t) __shfl_down(q, 3) & 0xffu;
    uint32_t      *run = ob + 12 * (t >> 5);
    if ((t & 3) == 0)
        run[(t & 31) >> 2] = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
    if ((t & 15) == 0) {
        run[8 + ((t >> 4) & 1)]  = __float_as_uint((float) sum);
        run[10 + ((t >> 4) & 1)] = __float_as_uint((float) (-32 * sum));
    }
}

/* the reciprocal of the row's scale from the row's largest magnitude, the scale to *o_scale */
__device__ __forceinline__ float q8s_row_inv(float ax, float *s_max, uint32_t *o_scale) {
    const int t = threadIdx.x;
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1)
        ax = __builtin_fmaxf(ax, __shfl_xor(ax, s));
    if ((t & 63) == 0)
        s_max[t >> 6] = ax;
    __syncthreads();
    const float amax = __builtin_fmaxf(__builtin_fmaxf(s_max[0], s_max[1]),
                                       __builtin_fmaxf(s_max[2], s_max[3]));
    float scale = __fdiv_rn(amax, 127.0f);
    if (scale == 0.0f)
        scale = 1.0f;
    if (t == 0)
        *o_scale = __float_as_uint(scale);
    return __fdiv_rn(1.0f, scale);
}

/* One workgroup per activation row. */
__global__ __launch_bounds__(Q6X_TPB) void k_q8s_row_quantize(const float *__restrict__ x, long ld_x,
                                                             int nb, uint32_t *__restrict__ act) {
    __shared__ float s_max[Q6X_TPB / 64];
    const int        m = blockIdx.x, t = threadIdx.x;
    const float     *xr = x + (long) m * ld_x;
    uint32_t        *o  = act + (long) m * ((long) nb * Q8K_ACT_DWORDS + Q8S_ACT_TAIL);
    float            ax = 0.0f;
    for (int b = 0; b < nb; ++b)
        ax = __builtin_fmaxf(ax, __builtin_fabsf(xr[256 * b + t])); /* (a NaN is passed over) */
    const float inv = q8s_row_inv(ax, s_max, o + (long) nb * Q8K_ACT_DWORDS);
    for (int b = 0; b < nb; ++b)
        q8s_quantize_block(xr[256 * b + t], inv, o + (long) b * Q8K_ACT_DWORDS);
}

/* The output norm (as k_rmsnorm_rows computes it) and that quantiser in one launch, one workgroup
 * per row; a thread reads back what it wrote itself. n a multiple of 256. */
__global__ __launch_bounds__(Q6X_TPB) void k_rmsnorm_q8s_rows(const float *__restrict__ x, long ld_x,
                                                             const float *__restrict__ w, float eps,
                                                             int n, float *__restrict__ y, long ld_y,
                                                             uint32_t *__restrict__ act) {
    __shared__ double s_part[Q6X_TPB];
    __shared__ float  s_inv;
    __shared__ float  s_max[Q6X_TPB / 64];
    const int    nb = n / 256, m = blockIdx.x, t = threadIdx.x;
    const float *xr = x + (long) m * ld_x;
    float       *yr = y + (long) m * ld_y;
    uint32_t    *o  = act + (long) m * ((long) nb * Q8K_ACT_DWORDS + Q8S_ACT_TAIL);
    const float  rinv = block_rms_inv<Q6X_TPB>(xr, n, eps, s_part, &s_inv);
    float        ax = 0.0f;
    for (int b = 0; b < nb; ++b) {
        const int   i = 256 * b + t;
        const float v = __fmul_rn(__fmul_rn(xr[i], rinv), w[i]);
        yr[i]         = v;
        ax            = __builtin_fmaxf(ax, __builtin_fabsf(v));
    }
    const float inv = q8s_row_inv(ax, s_max, o + (long) nb * Q8K_ACT_DWORDS);
    for (int b = 0; b < nb; ++b)
        q8s_quantize_block(yr[256 * b + t], inv, o + (long) b * Q8K_ACT_DWORDS);
}

typedef uint32_t q8s_u8v __attribute__((ext_vector_type(8), aligned(16)));

/* The rows grp * G .. of a step: each adds the run's two groups of sixteen to its accumulator.
 * z: the run's 32 values as bytes, four to a dword; ws0 / ws1: the groups' scales; av: the rows'
 * activations of the run; a_run: the run's twelve dwords of row 0. */
template <int M, int G, bool LANES>
__device__ __forceinline__ void q6x_group_rows(const uint32_t (&z)[8], float ws0, float ws1,
                                               const q8s_u8v (&av)[G],
                                               const uint32_t *__restrict__ a_run, long act_ld,
                                               int grp, float (&acc)[M]) {
    typedef float f2v __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int i = 0; i < G; ++i) {
        const int m = grp * G + i;
        if (m >= M)
            continue;
        const f2v sa = *reinterpret_cast<const f2v *>(a_run + m * act_ld + (LANES ? 10 : 8));
        int       d0 = 0, d1 = 0;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            d0 = __builtin_amdgcn_sdot4((int) z[u], (int) av[i][u], d0, false);
            d1 = __builtin_amdgcn_sdot4((int) z[4 + u], (int) av[i][4 + u], d1, false);
        }
        if (LANES) {
            acc[m] = __builtin_fmaf(ws0, (float) d0, acc[m]);
            acc[m] = __builtin_fmaf(ws0, sa[0], acc[m]);
            acc[m] = __builtin_fmaf(ws1, (float) d1, acc[m]);
            acc[m] = __builtin_fmaf(ws1, sa[1], acc[m]);
        } else {
            const float wo0 = __fmul_rn(ws0, 32.0f), wo1 = __fmul_rn(ws1, 32.0f);
            acc[m] = __fadd_rn(acc[m], __fsub_rn(__fmul_rn(ws0, (float) d0), __fmul_rn(wo0, sa[0])));
            acc[m] = __fadd_rn(acc[m], __fsub_rn(__fmul_rn(ws1, (float) d1), __fmul_rn(wo1, sa[1])));
        }
    }
}

/* M activation rows share a pass over the packed table. Steps of (run of 32 elements, group of up
 * to four rows): a run's eight fields are spread to bytes once; every row adds its own dot
 * products, with its activations as scalar operands that were loaded one step ahead, before the
 * fence that opens the step (an empty asm that loads may not pass and that needs the sums so
 * far: hoisted to the top of the block the rows' activations would not fit the scalar
 * registers). */
template <int M, bool LANES>
__global__ __launch_bounds__(Q6X_TPB, 4) void k_q6k_packed_gemm_x86(
    const uint32_t *__restrict__ packed, long n_out, int nb, const uint32_t *__restrict__ act,
    float *__restrict__ y, long ld_y) {
    typedef q8s_u8v u8v;
    constexpr int   G  = M < 4 ? M : 4;
    constexpr int NG = (M + G - 1) / G;
    const int     r  = threadIdx.x & 63;
    const long    g  = (long) blockIdx.x * (Q6X_TPB / 64) + threadIdx.x / 64;
    if (g * 64 >= n_out)
        return;
    const long row    = g * 64 + r;
    const long act_ld = (long) nb * Q8K_ACT_DWORDS + Q8S_ACT_TAIL;
    float      acc[M];
#pragma unroll
    for (int m = 0; m < M; ++m)
        acc[m] = 0.0f;
    /* loads run half a block ahead of the arithmetic, as in the decode kernel */
    const uint32_t *base = packed + g * nb * Q6X_PACK_DWORDS;
    uint32_t        qa[24], qb[24], sc[4], d52;
    q6x_load_scales(base, r, sc, d52);
    q6x_load6(base, r, 0, qa);
    for (int b = 0; b < nb; ++b) {
        const uint32_t *blk = base + (long) b * Q6X_PACK_DWORDS;
        const uint32_t *a   = act + (long) b * Q8K_ACT_DWORDS; /* uniform: scalar loads */
        q6x_load6(blk, r, 6, qb);
        const float    d         = __half2float(__ushort_as_half((unsigned short) (d52 & 0xffffu)));
        const uint32_t sc_now[4] = {sc[0], sc[1], sc[2], sc[3]};
        u8v            avc[G], avn[G];
#pragma unroll
        for (int i = 0; i < G; ++i)
            avc[i] = *reinterpret_cast<const u8v *>(a + i * act_ld);
        uint32_t z[8];
        float    ws0 = 0.0f, ws1 = 0.0f;
#pragma unroll
        for (int st = 0; st < 8 * NG; ++st) {
            const int v = st / NG, grp = st % NG; /* run v: elements 32 v .. 32 v + 31 */
            if (st + 1 < 8 * NG) {
                const int vn = (st + 1) / NG, gn = (st + 1) % NG;
#pragma unroll
                for (int i = 0; i < G; ++i)
                    if (gn * G + i < M)
                        avn[i] = *reinterpret_cast<const u8v *>(a + (gn * G + i) * act_ld + 12 * vn);
            }
#pragma unroll
            for (int i = 0; i < M; ++i)
                asm volatile("" : "+v"(acc[i])::"memory");
            if (st == 4 * NG && b + 1 < nb) { /* the first half's values are used up */
                q6x_load_scales(blk + Q6X_PACK_DWORDS, r, sc, d52);
                q6x_load6(blk + Q6X_PACK_DWORDS, r, 0, qa);
            }
            if (grp == 0) {
                const int vl = v & 3;
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    /* field f of the half: bits 24 f .. 24 f + 23 of its 24 dwords */
                    const int      f = 8 * vl + u, w0 = (3 * f) >> 2, sh = (3 * f) & 3;
                    const int      w1 = w0 + 1 < 24 ? w0 + 1 : 23;
                    const uint32_t lo = v < 4 ? qa[w0] : qb[w0], hi = v < 4 ? qa[w1] : qb[w1];
                    z[u] = sh == 0   ? q6x_spread<0>(lo, hi)
                           : sh == 1 ? q6x_spread<1>(lo, hi)
                           : sh == 2 ? q6x_spread<2>(lo, hi)
                                     : q6x_spread<3>(lo, hi);
                }
                ws0 = __fmul_rn(d, (float) q6x_scale(sc_now, 2 * v));
                ws1 = __fmul_rn(d, (float) q6x_scale(sc_now, 2 * v + 1));
            }
            q6x_group_rows<M, G, LANES>(z, ws0, ws1, avc, a + 12 * v, act_ld, grp, acc);
#pragma unroll
            for (int i = 0; i < G; ++i)
                avc[i] = avn[i];
        }
    }
    if (row < n_out) {
#pragma unroll
        for (int m = 0; m < M; ++m)
            y[m * ld_y + row] =
                __fmul_rn(__uint_as_float(act[m * act_ld + (long) nb * Q8K_ACT_DWORDS]), acc[m]);
    }
}

/* The same over the table as it lies in the file: a lane owns a table row and reads its 210-byte
 * blocks whole; a run's values come from ql and qh as in k_q6k_gemv_x86. */
template <int M, bool LANES>
__global__ __launch_bounds__(Q6X_TPB) void k_q6k_gemm_x86(const uint8_t *__restrict__ w, long n_out,
                                                          int nb, const uint32_t *__restrict__ act,
                                                          float *__restrict__ y, long ld_y) {
    typedef q8s_u8v u8v;
    constexpr int   G  = M < 4 ? M : 4;
    constexpr int   NG = (M + G - 1) / G;
    const long      row = (long) blockIdx.x * Q6X_TPB + threadIdx.x;
    if (row >= n_out)
        return;
    const uint8_t *rp     = w + row * (long) nb * 210;
    const long     act_ld = (long) nb * Q8K_ACT_DWORDS + Q8S_ACT_TAIL;
    float          acc[M];
#pragma unroll
    for (int m = 0; m < M; ++m)
        acc[m] = 0.0f;
    for (int b = 0; b < nb; ++b) {
        uint32_t dw[53];
        q6k_load_block(rp + (long) b * 210, dw);
        const uint32_t *a     = act + (long) b * Q8K_ACT_DWORDS; /* uniform: scalar loads */
        const uint32_t  sc[4] = {dw[48], dw[49], dw[50], dw[51]};
        const float     d = __half2float(__ushort_as_half((unsigned short) (dw[52] & 0xffffu)));
        u8v             avc[G], avn[G];
#pragma unroll
        for (int i = 0; i < G; ++i)
            avc[i] = *reinterpret_cast<const u8v *>(a + i * act_ld);
        uint32_t z[8];
        float    ws0 = 0.0f, ws1 = 0.0f;
#pragma unroll
        for (int st = 0; st < 8 * NG; ++st) {
            const int v = st / NG, grp = st % NG; /* run v = 4 h + j: elements 128 h + 32 j .. */
            if (st + 1 < 8 * NG) {
                const int vn = (st + 1) / NG, gn = (st + 1) % NG;
#pragma unroll
                for (int i = 0; i < G; ++i)
                    if (gn * G + i < M)
                        avn[i] = *reinterpret_cast<const u8v *>(a + (gn * G + i) * act_ld + 12 * vn);
            }
#pragma unroll
            for (int i = 0; i < M; ++i)
                asm volatile("" : "+v"(acc[i])::"memory");
            if (grp == 0) {
                const int h = v >> 2, j = v & 3;
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const uint32_t ql = dw[16 * h + 8 * (j & 1) + u], qh = dw[32 + 8 * h + u];
                    const uint32_t lo = (j >> 1) ? (ql >> 4) & 0x0f0f0f0fu : ql & 0x0f0f0f0fu;
                    const uint32_t hi = j == 0   ? (qh << 4) & 0x30303030u
                                        : j == 1 ? (qh << 2) & 0x30303030u
                                        : j == 2 ? qh & 0x30303030u
                                                 : (qh >> 2) & 0x30303030u;
                    z[u] = lo | hi;
                }
                ws0 = __fmul_rn(d, (float) q6x_scale(sc, 2 * v));
                ws1 = __fmul_rn(d, (float) q6x_scale(sc, 2 * v + 1));
            }
            q6x_group_rows<M, G, LANES>(z, ws0, ws1, avc, a + 12 * v, act_ld, grp, acc);
#pragma unroll
            for (int i = 0; i < G; ++i)
                avc[i] = avn[i];
        }
    }
#pragma unroll
    for (int m = 0; m < M; ++m)
        y[m * ld_y + row] =
            __fmul_rn(__uint_as_float(act[m * act_ld + (long) nb * Q8K_ACT_DWORDS]), acc[m]);
}

size_t q6k_x86_batch_act_dwords(int n_in) {
    return (size_t) (n_in / 256) * Q8K_ACT_DWORDS + Q8S_ACT_TAIL;
}

void launch_q8s_row_quantize(hipStream_t stream, const float *x, long ld_x, int n_m, int n_in,
                             uint32_t *act) {
    k_q8s_row_quantize<<<dim3(n_m), dim3(Q6X_TPB), 0, stream>>>(x, ld_x, n_in / 256, act);
}

void launch_rmsnorm_q8s_rows(hipStream_t stream, const float *x, long ld_x, const float *w,
                             float eps, int n_rows, int n, float *y, long ld_y, uint32_t *act) {
    k_rmsnorm_q8s_rows<<<dim3(n_rows), dim3(Q6X_TPB), 0, stream>>>(x, ld_x, w, eps, n, y, ld_y,
                                                                  act);
}

template <int M>
static void q6x_gemm_launch(hipStream_t stream, const void *table, bool packed, long n_out, int nb,
                            const uint32_t *act, bool lanes, float *y, long ld_y) {
    if (packed) {
        const uint32_t *p      = static_cast<const uint32_t *>(table);
        const long      groups = (n_out + 63) / 64;
        const dim3      grid((unsigned) ((groups + 3) / 4)), block(Q6X_TPB);
        if (lanes)
            k_q6k_packed_gemm_x86<M, true><<<grid, block, 0, stream>>>(p, n_out, nb, act, y, ld_y);
        else
            k_q6k_packed_gemm_x86<M, false><<<grid, block, 0, stream>>>(p, n_out, nb, act, y, ld_y);
    } else {
        const uint8_t *p = static_cast<const uint8_t *>(table);
        const dim3     grid((unsigned) ((n_out + Q6X_TPB - 1) / Q6X_TPB)), block(Q6X_TPB);
        if (lanes)
            k_q6k_gemm_x86<M, true><<<grid, block, 0, stream>>>(p, n_out, nb, act, y, ld_y);
        else
            k_q6k_gemm_x86<M, false><<<grid, block, 0, stream>>>(p, n_out, nb, act, y, ld_y);
    }
}

void launch_q6k_gemm_q8s(hipStream_t stream, const void *table, bool packed, long n_out, int n_in,
                         const uint32_t *act, int n_m, bool lanes, float *y, long ld_y) {
    const int nb = n_in / 256;
    switch (n_m) {
    case 1: q6x_gemm_launch<1>(stream, table, packed, n_out, nb, act, lanes, y, ld_y); break;
    case 2: q6x_gemm_launch<2>(stream, table, packed, n_out, nb, act, lanes, y, ld_y); break;
    case 3: q6x_gemm_launch<3>(stream, table, packed, n_out, nb, act, lanes, y, ld_y); break;
    case 4: q6x_gemm_launch<4>(stream, table, packed, n_out, nb, act, lanes, y, ld_y); break;
    case 5: q6x_gemm_launch<5>(stream, table, packed, n_out, nb, act, lanes, y, ld_y); break;
    case 6: q6x_gemm_launch<6>(stream, table, packed, n_out, nb, act, lanes, y, ld_y); break;
    case 7: q6x_gemm_launch<7>(stream, table, packed, n_out, nb, act, lanes, y, ld_y); break;
    default: q6x_gemm_launch<8>(stream, table, packed, n_out, nb, act, lanes, y, ld_y); break;
    }
}

void launch_q6k_gemv_q8k(hipStream_t stream, const uint8_t *w_q6k, long n_out, int n_in,
                         const uint32_t *act, float *y) {
    k_q6k_gemv_x86<<<dim3((unsigned) ((n_out + Q6X_TPB - 1) / Q6X_TPB)), dim3(Q6X_TPB), 0, stream>>>(
        w_q6k, n_out, n_in / 256, act, y);
}

void launch_q8k_quantize(hipStream_t stream, const float *x, long ld_x, int n_m, int n_in,
                         uint32_t *act) {
    const int nb = n_in / 256;
    k_q8k_quantize<<<dim3(nb, n_m), dim3(Q6X_TPB), 0, stream>>>(x, ld_x, nb, act);
}

void launch_rmsnorm_q8k_rows(hipStream_t stream, const float *x, long ld_x, const float *w,
                             float eps, int n_rows, int n, float *y, long ld_y, uint32_t *act) {
    k_rmsnorm_q8k_rows<<<dim3(n_rows), dim3(Q6X_TPB), 0, stream>>>(x, ld_x, w, eps, n, y, ld_y,
                                                                  act);
}

void launch_q6k_packed_gemv_q8k(hipStream_t stream, const void *packed, long n_out, int n_in,
                                const uint32_t *act, float *y) {
    const long groups = (n_out + 63) / 64;
    k_q6k_packed_gemv_x86<<<dim3((unsigned) ((groups + 3) / 4)), dim3(Q6X_TPB), 0, stream>>>(
        static_cast<const uint32_t *>(packed), n_out, n_in / 256, act, y);
}

} // namespace gs
