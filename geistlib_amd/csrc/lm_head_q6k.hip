/*
 * lm_head_q6k.hip -- the lm_head projection over a Q6_K table (gfx950), with the results of the
 * reference's portable kernels cpu_scalar_w_quant_m1 / _mN
 * (src/backends/cpu_scalar/weight_resolve.c:186-241) after dequant_q6_K_row
 * (src/formats/gguf/q6_K.c:13-45):
 *   y[m][r] = (float) sum_k (double) x[m][k] * (double) w[r][k]        (double, index order)
 *   w[r][k] = d * scale * (q - 32)                                     (binary32, left to right)
 * A Q6_K super-block is 256 elements in 210 bytes (src/quant/quant_blocks.h:67-73): ql[128],
 * qh[64], sixteen int8 scales, one binary16 d. Element 128 h + 32 j + l of a block has
 * q = nibble (j >> 1) of ql[64 h + 32 (j & 1) + l] | ((qh[32 h + l] >> 2 j) & 3) << 4 and the
 * scale 8 h + 2 j + l / 16.
 *
 * Arithmetic. d * scale has at most 11 + 8 significant bits and (q - 32) at most 6, so both
 * binary32 products of the dequantisation are exact, and so is every product x * w in double
 * (24 + 24 bits): the reference's result is the exact sum of the products but for the rounding
 * of its 1 + n_in additions. Here a lane owns a table row. It adds, per group of 16 elements
 * that share a scale, t = sum x * q_unsigned in double (exact products again), and then
 * ds * (t - 32 * sum x) to the row's sum, ds = d * scale; the sums of x and |x| per group come
 * with the double copy of the activations. The result differs from the reference's by at most
 *   err = 2^-53 * (32 * sum_g (n_in - 16 g) |ds_g| X_g  +  (1700 + 96 n_g) * sum_g |ds_g| X_g),
 * X_g = sum |x| over group g: the first term bounds the rounding of the reference's sequential
 * additions (the k-th addition's error is at most 2^-53 times the sum of the |products| so
 * far, and |w| <= 32 |ds|), the second everything this kernel rounds (16 additions per group on
 * values below 63 X_g, the subtraction, the product with ds, one addition per group of the row's
 * sum, n_g = n_in / 16 of them). When every value within err of the sum rounds to the same
 * binary32 the reference's result is that binary32; otherwise -- a few outputs in ten thousand -- the output goes on a
 * list and a second kernel adds its products once more one after the other in index order.
 *
 * Memory. A lane reads its row's blocks with aligned 16-byte loads straight from the table:
 * consecutive loads of a lane use up the cache lines that its first load fetched, and all bytes
 * of the table are read once. Blocks start on 2-byte boundaries; a block is fetched as the 53
 * aligned dwords that hold it and shifted into place. The activations are uniform over the
 * wavefront and come as scalar operands.
 */
#include "lm_head_kernels.h"
#include "lm_head_q6k_block.h"

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gs {

constexpr int Q6K_BLOCK_BYTES = 210;
constexpr int Q6K_BLOCK_ELEMS = 256;
constexpr int Q6K_TPB         = 256;

/* (float) s, and whether every value within err of s rounds to the same binary32. */
__device__ __forceinline__ bool q6k_rounding_is_safe(double s, double err, float &f) {
    f = (float) s;
    /* Not finite: with an infinite or NaN activation the sum's terms are infinities and NaNs,
     * and this kernel's split into t - 32 * sum x can meet inf - inf where the reference's sum in
     * index order does not. The kernel that adds in the reference's order decides. */
    if (!(__builtin_fabsf(f) < __builtin_inff()))
        return false;
    const double up = 0.5 * ((double) f + (double) nextafterf(f, __builtin_inff()));
    const double dn = 0.5 * ((double) f + (double) nextafterf(f, -__builtin_inff()));
    return up - s > err && s - dn > err;
}

/* xd[m][k] = (double) x[m][k]; per group of 16 elements xsum = sum x and xabs = sum |x| (rounded
 * up); the count of listed outputs starts at zero. One workgroup per activation row. */
__global__ __launch_bounds__(Q6K_TPB) void k_q6k_x_prep(const float *__restrict__ x, long ld_x,
                                                        int n_in, double *__restrict__ xd,
                                                        double *__restrict__ xsum,
                                                        double *__restrict__ xabs,
                                                        int *amb_count) {
    const int    m  = blockIdx.x;
    const float *xr = x + (long) m * ld_x;
    if (m == 0 && threadIdx.x == 0)
        *amb_count = 0;
    for (int k = threadIdx.x; k < n_in; k += Q6K_TPB)
        xd[(long) m * n_in + k] = (double) xr[k];
    const int n_g = n_in / 16;
    for (int g = threadIdx.x; g < n_g; g += Q6K_TPB) {
        double s = 0.0, a = 0.0;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const double v = (double) xr[16 * g + i];
            s += v;
            a += __builtin_fabs(v);
        }
        xsum[(long) m * n_g + g] = s;
        xabs[(long) m * n_g + g] = a * (1.0 + 0x1p-40);
    }
}

/* byte i of v as a float (one conversion instruction per byte) */
__device__ __forceinline__ float q6k_ubyte(uint32_t v, int i) {
    return (float) ((v >> (8 * i)) & 0xffu);
}

template <int MT>
__global__ __launch_bounds__(Q6K_TPB) void k_q6k_linear(const uint8_t *__restrict__ w, long n_out,
                                                        int n_in, const double *__restrict__ xd,
                                                        const double *__restrict__ xsum,
                                                        const double *__restrict__ xabs, int n_m,
                                                        float *__restrict__ y, long ld_y,
                                                        int *__restrict__ amb_count,
                                                        int2 *__restrict__ amb_list) {
    const long row = (long) blockIdx.x * Q6K_TPB + threadIdx.x;
    if (row >= n_out)
        return;
    const int      nb  = n_in / Q6K_BLOCK_ELEMS, n_g = n_in / 16;
    const uint8_t *rp  = w + row * (long) nb * Q6K_BLOCK_BYTES;
    double         S[MT], B[MT], Bw[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
        S[m] = B[m] = Bw[m] = 0.0;
    for (int b = 0; b < nb; ++b) {
        uint32_t d[53];
        q6k_load_block(rp + (long) b * Q6K_BLOCK_BYTES, d);
        const float dd = __half2float(__ushort_as_half((unsigned short) (d[52] & 0xffffu)));
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int is = 0; is < 2; ++is) {
                double t[4][MT];
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int m = 0; m < MT; ++m)
                        t[j][m] = 0.0;
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const uint32_t ql_a = d[16 * h + 4 * is + s];
                    const uint32_t ql_b = d[16 * h + 8 + 4 * is + s];
                    const uint32_t qh4  = d[32 + 8 * h + 4 * is + s];
                    uint32_t       qu[4]; /* the unsigned 6-bit values of four elements, a byte each */
                    qu[0] = (ql_a & 0x0F0F0F0Fu) | ((qh4 << 4) & 0x30303030u);
                    qu[1] = (ql_b & 0x0F0F0F0Fu) | ((qh4 << 2) & 0x30303030u);
                    qu[2] = ((ql_a >> 4) & 0x0F0F0F0Fu) | (qh4 & 0x30303030u);
                    qu[3] = ((ql_b >> 4) & 0x0F0F0F0Fu) | ((qh4 >> 2) & 0x30303030u);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        /* elements 256 b + 128 h + 32 j + 16 is + 4 s + i */
                        const int k0 = Q6K_BLOCK_ELEMS * b + 128 * h + 32 * j + 16 * is + 4 * s;
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const double q = (double) q6k_ubyte(qu[j], i);
#pragma unroll
                            for (int m = 0; m < MT; ++m) {
                                const double *xm = xd + (long) (m < n_m ? m : n_m - 1) * n_in;
                                t[j][m] = __builtin_fma(xm[k0 + i], q, t[j][m]); /* uniform address */
                            }
                        }
                    }
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int    si = 8 * h + 2 * j + is; /* scale of the group within the block */
                    const int    sc = (int) (int8_t) (d[48 + si / 4] >> (8 * (si % 4)));
                    const double ds = (double) (dd * (float) sc);
                    const int    g  = 16 * b + si;        /* the group's place in the row */
                    const double pos = (double) (n_in - 16 * g);
#pragma unroll
                    for (int m = 0; m < MT; ++m) {
                        const long   at = (long) (m < n_m ? m : n_m - 1) * n_g + g;
                        const double v  = __builtin_fma(-32.0, xsum[at], t[j][m]);
                        S[m]            = __builtin_fma(ds, v, S[m]);
                        const double bx = __builtin_fabs(ds) * xabs[at];
                        B[m] += bx;
                        Bw[m] = __builtin_fma(pos, bx, Bw[m]);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        if (m < n_m) {
            const double err =
                0x1p-53 * (32.0 * Bw[m] + (1700.0 + 96.0 * n_g) * B[m]) * (1.0 + 0x1p-30);
            float        f;
            if (!q6k_rounding_is_safe(S[m], err, f))
                amb_list[atomicAdd(amb_count, 1)] = make_int2((int) row, m);
            y[m * ld_y + row] = f;
        }
    }
}

/* The listed outputs once more, the products added one after the other in index order as the
 * reference adds them. A wavefront per output (table row r, activation row m): its lanes form 64
 * products at a time -- each exact in double, whichever way it is computed -- and the sum takes
 * them in order, lane by lane, as scalar operands. The chain of n_in dependent additions
 * is what this kernel takes; there are few listed outputs and each has a wavefront to itself. */
constexpr int Q6K_LISTED_WAVES = 4;
__global__ __launch_bounds__(64 * Q6K_LISTED_WAVES) void k_q6k_linear_listed(
    const uint8_t *__restrict__ w, int n_in, const double *__restrict__ xd, float *__restrict__ y,
    long ld_y, const int *__restrict__ amb_count, const int2 *__restrict__ amb_list) {
    const int count = *amb_count;
    const int nb    = n_in / Q6K_BLOCK_ELEMS;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int it0 = blockIdx.x * Q6K_LISTED_WAVES; it0 < count;
         it0 += gridDim.x * Q6K_LISTED_WAVES) {
        const int      it   = it0 + wave < count ? it0 + wave : count - 1;
        const int2     mine = amb_list[it];
        const uint8_t *rp   = w + (long) mine.x * nb * Q6K_BLOCK_BYTES;
        const double  *xm   = xd + (long) mine.y * n_in;
        double         acc  = 0.0;
        for (int b = 0; b < nb; ++b) {
            /* the four 64-element rounds of a block: their loads first, all in flight together */
            const uint8_t *p = rp + (long) b * Q6K_BLOCK_BYTES;
            const int      l = lane & 31;
            const float    dd = __half2float(
                __ushort_as_half((unsigned short) (p[208] | ((unsigned) p[209] << 8))));
            double prod[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) { /* element 64 r + lane: h = r / 2, j = 2 (r & 1) + lane / 32 */
                const int      h = r >> 1, j = 2 * (r & 1) + (lane >> 5);
                const uint32_t lo = p[64 * h + 32 * (j & 1) + l];
                const int      q  = (int) (((j >> 1) ? lo >> 4 : lo & 0xFu) |
                                          (((p[128 + 32 * h + l] >> (2 * j)) & 3u) << 4)) - 32;
                const int   sc = (int) (int8_t) p[192 + 8 * h + 2 * j + l / 16];
                const float wv = dd * (float) sc * (float) q; /* q6_K.c:37-40 */
                prod[r]        = xm[Q6K_BLOCK_ELEMS * b + 64 * r + lane] * (double) wv;
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                /* lane i's product as a scalar operand, i = 0 .. 63 in order: the additions are
                 * the only dependent chain (every lane runs it; the first lane's copy is used) */
                const uint2 pw = __builtin_bit_cast(uint2, prod[r]);
#pragma unroll
                for (int i = 0; i < 64; ++i) {
                    uint2 t;
                    t.x = (uint32_t) __builtin_amdgcn_readlane((int) pw.x, i);
                    t.y = (uint32_t) __builtin_amdgcn_readlane((int) pw.y, i);
                    acc += __builtin_bit_cast(double, t);
                }
            }
        }
        if (lane == 0 && it0 + wave < count)
            y[mine.y * ld_y + mine.x] = (float) acc;
    }
}

/* ---- the table repacked for the device --------------------------------------------------------
 * The GGUF layout puts a row's blocks one after the other, 210 bytes each: lanes that own
 * neighbouring rows read addresses a row apart, a block shares its first and last cache line
 * with its neighbours, and an element's six bits lie in two places. geist_hip_q6k_pack (once per
 * model, at load) writes the same information in the order and form the kernel wants: the table
 * rows in groups of 64 (a wavefront), per group the blocks in order, per block 53 dwords for
 * each of the 64 rows with the rows innermost --
 *   dwords 4 p .. 4 p + 3 of row r (p < 13) at  base + p * 256 + 4 r,   dword 52 at base + 3328 + r
 * (in dwords; base = (group * blocks + b) * 3392) -- so that a wavefront's 16-byte loads read one
 * kilobyte of consecutive addresses and every byte is read once. A row's 53 dwords hold the
 * block's 256 six-bit values in the order of the elements, element e in bits 6 e .. 6 e + 5 of
 * dwords 0..47 (one extraction per element; two of every sixteen straddle a dword), the sixteen
 * scales in dwords 48..51 and d in the low half of dword 52. Rows beyond n_out in the last group
 * are zero blocks.
 *
 * With the loads and the bit assembly out of the way the kernel can afford the reference's own
 * order of additions: a lane owns a table row and adds its products one after the other in index
 * order,
 *   acc = fma(x[k], w[k], acc),  w = fma(ds, q_unsigned, -32 ds)   (both exact, see the header)
 * which is cpu_scalar_w_quant_m1's sum bit for bit, with nothing to bound and nothing to repeat.
 * The chain of dependent additions is hidden by the conversions of the following elements and
 * by the other wavefronts of the SIMD. */
constexpr int Q6K_PACK_DWORDS = 53 * 64; /* per (group of 64 rows, block) */

__global__ __launch_bounds__(Q6K_TPB) void k_q6k_pack(const uint8_t *__restrict__ w, long n_out,
                                                      int nb, uint32_t *__restrict__ packed) {
    const long item = (long) blockIdx.x * (Q6K_TPB / 64) + threadIdx.x / 64; /* (group, block) */
    const int  r    = threadIdx.x & 63;
    const long n_groups = (n_out + 63) / 64;
    if (item >= n_groups * nb)
        return;
    const long g = item / nb, row = g * 64 + r;
    const int  b = (int) (item - g * nb);
    uint32_t   d[53];
    if (row < n_out) {
        q6k_load_block(w + (row * nb + b) * (long) Q6K_BLOCK_BYTES, d);
        d[52] &= 0xffffu;
    } else {
#pragma unroll
        for (int i = 0; i < 53; ++i)
            d[i] = 0u;
    }
    /* the six-bit values in element order: element 128 h + 32 j + l takes nibble (j >> 1) of
     * ql[64 h + 32 (j & 1) + l] and bits 2 j, 2 j + 1 of qh[32 h + l] (q6_K.c:30-36) */
    uint32_t o[53];
#pragma unroll
    for (int i = 0; i < 48; ++i)
        o[i] = 0u;
#pragma unroll
    for (int e = 0; e < 256; ++e) {
        const int      h = e >> 7, j = (e >> 5) & 3, l = e & 31;
        const int      qlb = 64 * h + 32 * (j & 1) + l, qhb = 32 * h + l;
        const uint32_t lo = (d[qlb / 4] >> (8 * (qlb % 4) + 4 * (j >> 1))) & 0xFu;
        const uint32_t hi = (d[32 + qhb / 4] >> (8 * (qhb % 4) + 2 * j)) & 3u;
        const uint32_t q  = lo | (hi << 4);
        const int      bit = 6 * e, w0 = bit >> 5, off = bit & 31;
        o[w0] |= q << off;
        if (off > 26)
            o[w0 + 1] |= q >> (32 - off);
    }
#pragma unroll
    for (int i = 48; i < 53; ++i)
        o[i] = d[i];
    uint32_t *base = packed + item * Q6K_PACK_DWORDS;
#pragma unroll
    for (int p = 0; p < 13; ++p)
        *reinterpret_cast<uint4 *>(base + p * 256 + 4 * r) =
            make_uint4(o[4 * p], o[4 * p + 1], o[4 * p + 2], o[4 * p + 3]);
    base[3328 + r] = o[52];
}

/* six of a lane's 16-byte pieces of a packed block, from piece p0 on: 24 dwords, the six-bit
 * values of half a block */
__device__ __forceinline__ void q6k_packed_load6(const uint32_t *__restrict__ base, int r, int p0,
                                                 uint32_t (&q)[24]) {
#pragma unroll
    for (int p = 0; p < 6; ++p) {
        typedef uint32_t nt_u4 __attribute__((ext_vector_type(4)));
        const nt_u4 t = __builtin_nontemporal_load(
            reinterpret_cast<const nt_u4 *>(base + (p0 + p) * 256 + 4 * r));
        q[4 * p] = t.x, q[4 * p + 1] = t.y, q[4 * p + 2] = t.z, q[4 * p + 3] = t.w;
    }
}
/* the sixteen scales (four dwords) and d of a lane's block */
__device__ __forceinline__ void q6k_packed_load_scales(const uint32_t *__restrict__ base, int r,
                                                       uint32_t (&sc)[4], uint32_t &d52) {
    typedef uint32_t nt_u4 __attribute__((ext_vector_type(4)));
    const nt_u4 t =
        __builtin_nontemporal_load(reinterpret_cast<const nt_u4 *>(base + 12 * 256 + 4 * r));
    sc[0] = t.x, sc[1] = t.y, sc[2] = t.z, sc[3] = t.w;
    d52   = __builtin_nontemporal_load(base + 3328 + r);
}
/* acc[m] += the 128 products of half a block with activation row m, one after the other in
 * index order; `q` the half's six-bit values, `sc_lo`, `sc_hi` its eight scales, `x0` the
 * half's first activation of row 0 */
template <int MT>
__device__ __forceinline__ void q6k_packed_half(uint32_t (&q)[24], uint32_t sc_lo,
                                                uint32_t sc_hi, float dd,
                                                const double *__restrict__ x0, int n_m, int n_in,
                                                double (&acc)[MT]) {
#pragma unroll
    for (int g16 = 0; g16 < 8; ++g16) { /* eight scale groups, in element order */
        const int    sc = (int) (int8_t) ((g16 < 4 ? sc_lo : sc_hi) >> (8 * (g16 % 4)));
        const double ds = (double) (dd * (float) sc), m32ds = -32.0 * ds;
        const double *xg = x0 + 16 * g16;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int bit = 6 * (16 * g16 + i), w0 = bit >> 5, off = bit & 31;
            /* (straddling values: the funnel shift's low six bits) */
            const uint32_t v  = off <= 26
                                    ? (q[w0] >> off) & 63u
                                    : __builtin_amdgcn_alignbit(q[w0 + 1 < 24 ? w0 + 1 : 23], q[w0],
                                                                off) & 63u;
            const double   wv = __builtin_fma(ds, (double) v, m32ds);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const double *xm = xg + (long) (m < n_m ? m : n_m - 1) * n_in;
                acc[m] = __builtin_fma(xm[i], wv, acc[m]); /* uniform address */
            }
        }
        /* one scale group at a time: left alone the scheduler converts far ahead and runs out of
         * registers. The empty asm makes the next group's three dwords wait for this group's
         * sum. */
        if (g16 + 1 < 8) {
            asm volatile("" : "+v"(acc[0]), "+v"(q[3 * g16 + 3]), "+v"(q[3 * g16 + 4]),
                              "+v"(q[3 * g16 + 5]));
        }
    }
}

template <int MT>
__global__ __launch_bounds__(Q6K_TPB, 4) void k_q6k_packed_linear(const uint32_t *__restrict__ packed,
                                                               long n_out, int n_in,
                                                               const double *__restrict__ xd,
                                                               int n_m, float *__restrict__ y,
                                                               long ld_y) {
    const int  r = threadIdx.x & 63;
    const long g = (long) blockIdx.x * (Q6K_TPB / 64) + threadIdx.x / 64;
    if (g * 64 >= n_out)
        return;
    const long row = g * 64 + r;
    const int  nb  = n_in / Q6K_BLOCK_ELEMS;
    double     acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
        acc[m] = 0.0;
    /* Loads run half a block ahead of the arithmetic (a wavefront has few neighbours on its SIMD
     * to cover a wait: the whole table is 4 wavefronts per SIMD): a block's second half is asked
     * for when its first half is about to be added up, the next block's first half and scales
     * when this block's second half is. */
    const uint32_t *base = packed + g * nb * Q6K_PACK_DWORDS;
    uint32_t        qa[24], qb[24], sc[4], d52;
    q6k_packed_load_scales(base, r, sc, d52);
    q6k_packed_load6(base, r, 0, qa);
    for (int b = 0; b < nb; ++b) {
        const uint32_t *blk = base + (long) b * Q6K_PACK_DWORDS;
        const double   *x0  = xd + (long) b * Q6K_BLOCK_ELEMS;
        q6k_packed_load6(blk, r, 6, qb);
        const float    dd  = __half2float(__ushort_as_half((unsigned short) (d52 & 0xffffu)));
        const uint32_t sc2 = sc[2], sc3 = sc[3];
        q6k_packed_half<MT>(qa, sc[0], sc[1], dd, x0, n_m, n_in, acc);
        if (b + 1 < nb) {
            q6k_packed_load_scales(blk + Q6K_PACK_DWORDS, r, sc, d52);
            q6k_packed_load6(blk + Q6K_PACK_DWORDS, r, 0, qa);
        }
        q6k_packed_half<MT>(qb, sc2, sc3, dd, x0 + 128, n_m, n_in, acc);
    }
    if (row < n_out) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
            if (m < n_m)
                y[m * ld_y + row] = (float) acc[m];
    }
}

/* Several activation rows at once: a block at a time, every weight converted once and used for
 * each row (the scalar registers that hold the rows' activations leave no room for running the
 * loads ahead). */
template <int MT>
__global__ __launch_bounds__(Q6K_TPB) void k_q6k_packed_linear_rows(const uint32_t *__restrict__ packed,
                                                               long n_out, int n_in,
                                                               const double *__restrict__ xd,
                                                               int n_m, float *__restrict__ y,
                                                               long ld_y) {
    const int  r = threadIdx.x & 63;
    const long g = (long) blockIdx.x * (Q6K_TPB / 64) + threadIdx.x / 64;
    if (g * 64 >= n_out)
        return;
    const long row = g * 64 + r;
    const int  nb  = n_in / Q6K_BLOCK_ELEMS;
    double     acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
        acc[m] = 0.0;
    for (int b = 0; b < nb; ++b) {
        const uint32_t *base = packed + (g * nb + b) * Q6K_PACK_DWORDS;
        uint32_t        d[53];
#pragma unroll
        for (int p = 0; p < 13; ++p) {
            typedef uint32_t nt_u4 __attribute__((ext_vector_type(4)));
            const nt_u4 q = __builtin_nontemporal_load(
                reinterpret_cast<const nt_u4 *>(base + p * 256 + 4 * r));
            d[4 * p] = q.x, d[4 * p + 1] = q.y, d[4 * p + 2] = q.z, d[4 * p + 3] = q.w;
        }
        d[52] = __builtin_nontemporal_load(base + 3328 + r);
        const float dd = __half2float(__ushort_as_half((unsigned short) (d[52] & 0xffffu)));
#pragma unroll
        for (int g16 = 0; g16 < 16; ++g16) { /* the sixteen scale groups, in element order */
            const int    sc = (int) (int8_t) (d[48 + g16 / 4] >> (8 * (g16 % 4)));
            const double ds = (double) (dd * (float) sc), m32ds = -32.0 * ds;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int bit = 6 * (16 * g16 + i), w0 = bit >> 5, off = bit & 31;
                /* (straddling values: the funnel shift's low six bits) */
                const uint32_t q  = off <= 26
                                        ? (d[w0] >> off) & 63u
                                        : __builtin_amdgcn_alignbit(d[w0 + 1], d[w0], off) & 63u;
                const double   wv = __builtin_fma(ds, (double) q, m32ds);
                const int      k  = Q6K_BLOCK_ELEMS * b + 16 * g16 + i;
#pragma unroll
                for (int m = 0; m < MT; ++m) {
                    const double *xm = xd + (long) (m < n_m ? m : n_m - 1) * n_in;
                    acc[m] = __builtin_fma(xm[k], wv, acc[m]); /* uniform address */
                }
            }
        }
    }
    if (row < n_out) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
            if (m < n_m)
                y[m * ld_y + row] = (float) acc[m];
    }
}

size_t q6k_packed_bytes(long n_out, int n_in) {
    return (size_t) ((n_out + 63) / 64) * (size_t) (n_in / Q6K_BLOCK_ELEMS) * Q6K_PACK_DWORDS * 4;
}

void launch_q6k_pack(hipStream_t stream, const uint8_t *w_q6k, long n_out, int n_in,
                     void *packed) {
    const int  nb    = n_in / Q6K_BLOCK_ELEMS;
    const long items = (n_out + 63) / 64 * nb;
    k_q6k_pack<<<dim3((unsigned) ((items + 3) / 4)), dim3(Q6K_TPB), 0, stream>>>(
        w_q6k, n_out, nb, static_cast<uint32_t *>(packed));
}

void launch_q6k_packed_linear(hipStream_t stream, const void *packed, long n_out, int n_in,
                              const float *x, long ld_x, int n_m, const Q6KScratch &ws, float *y,
                              long ld_y) {
    k_q6k_x_prep<<<dim3(n_m), dim3(Q6K_TPB), 0, stream>>>(x, ld_x, n_in, ws.xd, ws.xsum, ws.xabs,
                                                         ws.amb_count);
    const long     groups = (n_out + 63) / 64;
    const dim3     grid((unsigned) ((groups + 3) / 4)), block(Q6K_TPB);
    const uint32_t *p = static_cast<const uint32_t *>(packed);
    switch (n_m) {
    case 1: k_q6k_packed_linear<1><<<grid, block, 0, stream>>>(p, n_out, n_in, ws.xd, n_m, y, ld_y); break;
    case 2: k_q6k_packed_linear_rows<2><<<grid, block, 0, stream>>>(p, n_out, n_in, ws.xd, n_m, y, ld_y); break;
    default: k_q6k_packed_linear_rows<4><<<grid, block, 0, stream>>>(p, n_out, n_in, ws.xd, n_m, y, ld_y); break;
    }
}

void launch_q6k_linear(hipStream_t stream, const uint8_t *w_q6k, long n_out, int n_in,
                       const float *x, long ld_x, int n_m, const Q6KScratch &ws, float *y,
                       long ld_y) {
    k_q6k_x_prep<<<dim3(n_m), dim3(Q6K_TPB), 0, stream>>>(x, ld_x, n_in, ws.xd, ws.xsum, ws.xabs,
                                                         ws.amb_count);
    const dim3 grid((unsigned) ((n_out + Q6K_TPB - 1) / Q6K_TPB)), block(Q6K_TPB);
    switch (n_m) {
    case 1:
        k_q6k_linear<1><<<grid, block, 0, stream>>>(w_q6k, n_out, n_in, ws.xd, ws.xsum, ws.xabs,
                                                    n_m, y, ld_y, ws.amb_count, ws.amb_list);
        break;
    case 2:
        k_q6k_linear<2><<<grid, block, 0, stream>>>(w_q6k, n_out, n_in, ws.xd, ws.xsum, ws.xabs,
                                                    n_m, y, ld_y, ws.amb_count, ws.amb_list);
        break;
    default:
        k_q6k_linear<4><<<grid, block, 0, stream>>>(w_q6k, n_out, n_in, ws.xd, ws.xsum, ws.xabs,
                                                    n_m, y, ld_y, ws.amb_count, ws.amb_list);
        break;
    }
    /* the list is short (a few outputs in ten thousand) but its length is only known on the
     * device: a workgroup per four listed outputs for up to one output in 256, most of which
     * return at once; longer lists (rows that cancel) go round the loop */
    const long     want_wgs   = ((long) n_out * n_m / 256 + Q6K_LISTED_WAVES - 1) / Q6K_LISTED_WAVES + 1;
    const unsigned listed_wgs = (unsigned) (want_wgs < 2048 ? want_wgs : 2048);
    k_q6k_linear_listed<<<dim3(listed_wgs), dim3(64 * Q6K_LISTED_WAVES), 0, stream>>>(
        w_q6k, n_in, ws.xd, y, ld_y, ws.amb_count, ws.amb_list);
}


/* ==== Q4_K ==================================================================================
 * Super-blocks of 144 bytes: d and dmin (binary16), eight 6-bit scales and eight 6-bit minima
 * in 12 bytes, 128 bytes of 4-bit values (src/quant/quant_blocks.h:50-56). dequant_q4_K_row
 * (src/formats/gguf/q4_K.c:18-49): element 64 s + l of a block is
 *   (d * sc[2 s]) * (qs[32 s + l] & 15) - dmin * m[2 s],
 * element 64 s + 32 + l the same with the high nibble and sc / m[2 s + 1]. d * sc (11 + 6 bits)
 * and its product with the 4-bit value are exact in binary32, so the element is one rounding
 * of an exact difference: a fused multiply-add gives the reference's bits whether or not its
 * compiler contracted the expression. The projection adds (double) x * (double) w in index
 * order (cpu_scalar_w_quant_m1 / _mN), as for Q6_K.
 *
 * Only the packed form has a kernel. geist_hip_q4k_pack writes, per group of 64 table rows and
 * block, 37 dwords for each row with the rows innermost (dwords 4 p .. 4 p + 3 of row r, p < 9,
 * at base + p * 256 + 4 r, dword 36 at base + 2304 + r; base = (group * blocks + b) * 2368):
 * dwords 0..31 the 4-bit values in element order (element e in bits 4 (e % 8) .. of dword e / 8),
 * 32..33 the eight scales and 34..35 the eight minima as bytes, 36 d (low half) and dmin. 148
 * bytes for a block's 144: the 6-bit fields are spread to bytes once, at load.
 * ========================================================================================== */
constexpr int Q4K_BLOCK_BYTES = 144;
constexpr int Q4K_ROW_DWORDS  = 37;
constexpr int Q4K_PACK_DWORDS = Q4K_ROW_DWORDS * 64;

__global__ __launch_bounds__(Q6K_TPB) void k_q4k_pack(const uint8_t *__restrict__ w, long n_out,
                                                      int nb, uint32_t *__restrict__ packed) {
    const int  r    = threadIdx.x & 63;
    const long item = (long) blockIdx.x * (Q6K_TPB / 64) + threadIdx.x / 64; /* (group, block) */
    const long g    = item / nb;
    const int  b    = (int) (item % nb);
    if (g * 64 >= n_out)
        return;
    const long row = g * 64 + r;
    uint32_t   d[36]; /* the block's 144 bytes; a row beyond the table is a block of zeros */
#pragma unroll
    for (int i = 0; i < 36; ++i)
        d[i] = 0u;
    if (row < n_out) {
        const uint8_t *src = w + ((size_t) row * nb + b) * Q4K_BLOCK_BYTES; /* 4-byte aligned: 144 = 36 * 4 */
        const uint32_t *s4 = reinterpret_cast<const uint32_t *>(src);
#pragma unroll
        for (int i = 0; i < 36; ++i)
            d[i] = s4[i];
    }
    uint32_t o[Q4K_ROW_DWORDS];
    /* bytes 16 + 32 s + l hold elements 64 s + l (low nibble) and 64 s + 32 + l (high) */
#pragma unroll
    for (int i = 0; i < 32; ++i)
        o[i] = 0u;
#pragma unroll
    for (int e = 0; e < 256; ++e) {
        const int      s = e >> 6, hi = (e >> 5) & 1, l = e & 31;
        const int      byte = 16 + 32 * s + l;
        const uint32_t q = (d[byte / 4] >> (8 * (byte % 4) + 4 * hi)) & 0xFu;
        o[e >> 3] |= q << (4 * (e & 7));
    }
    /* get_scale_min_k4 (quant_blocks.h:103-111) over the 12 bytes at offset 4 */
    auto sbyte = [&](int i) { return (d[1 + i / 4] >> (8 * (i % 4))) & 0xFFu; };
    o[32] = o[33] = o[34] = o[35] = 0u;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        uint32_t sc, mn;
        if (j < 4) {
            sc = sbyte(j) & 63u;
            mn = sbyte(j + 4) & 63u;
        } else {
            sc = (sbyte(j + 4) & 0xFu) | ((sbyte(j - 4) >> 6) << 4);
            mn = (sbyte(j + 4) >> 4) | ((sbyte(j) >> 6) << 4);
        }
        o[32 + j / 4] |= sc << (8 * (j % 4));
        o[34 + j / 4] |= mn << (8 * (j % 4));
    }
    o[36] = d[0]; /* d, dmin */
    uint32_t *base = packed + item * Q4K_PACK_DWORDS;
#pragma unroll
    for (int p = 0; p < 9; ++p)
        *reinterpret_cast<uint4 *>(base + p * 256 + 4 * r) =
            make_uint4(o[4 * p], o[4 * p + 1], o[4 * p + 2], o[4 * p + 3]);
    base[2304 + r] = o[36];
}

/* A lane owns a table row and adds its products one after the other in index order. Per weight:
 * its byte (the nibbles of a dword are spread to bytes by two masks for eight weights), the
 * conversion, one fused multiply-add in binary32 (the element), its conversion to double, one
 * in double (the sum). */
template <int MT>
__global__ __launch_bounds__(Q6K_TPB) void k_q4k_packed_linear(const uint32_t *__restrict__ packed,
                                                               long n_out, int n_in,
                                                               const double *__restrict__ xd,
                                                               int n_m, float *__restrict__ y,
                                                               long ld_y) {
    const int  r = threadIdx.x & 63;
    const long g = (long) blockIdx.x * (Q6K_TPB / 64) + threadIdx.x / 64;
    if (g * 64 >= n_out)
        return;
    const long row = g * 64 + r;
    const int  nb  = n_in / Q6K_BLOCK_ELEMS;
    double     acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
        acc[m] = 0.0;
    for (int b = 0; b < nb; ++b) {
        const uint32_t *base = packed + (g * nb + b) * Q4K_PACK_DWORDS;
        uint32_t        d[Q4K_ROW_DWORDS];
        /* scales, minima and d first: the arithmetic can start when they and the first values
         * have arrived */
        {
            typedef uint32_t nt_u4 __attribute__((ext_vector_type(4)));
            const nt_u4 q = __builtin_nontemporal_load(
                reinterpret_cast<const nt_u4 *>(base + 8 * 256 + 4 * r));
            d[32] = q.x, d[33] = q.y, d[34] = q.z, d[35] = q.w;
            d[36] = __builtin_nontemporal_load(base + 2304 + r);
        }
#pragma unroll
        for (int p = 0; p < 8; ++p) {
            typedef uint32_t nt_u4 __attribute__((ext_vector_type(4)));
            const nt_u4 q = __builtin_nontemporal_load(
                reinterpret_cast<const nt_u4 *>(base + p * 256 + 4 * r));
            d[4 * p] = q.x, d[4 * p + 1] = q.y, d[4 * p + 2] = q.z, d[4 * p + 3] = q.w;
        }
        const float dd   = __half2float(__ushort_as_half((unsigned short) (d[36] & 0xffffu)));
        const float dmin = __half2float(__ushort_as_half((unsigned short) (d[36] >> 16)));
#pragma unroll
        for (int j = 0; j < 8; ++j) { /* the eight sub-blocks of 32 elements */
            const float d1  = dd * (float) ((d[32 + j / 4] >> (8 * (j % 4))) & 0xFFu);
            const float nm1 = -(dmin * (float) ((d[34 + j / 4] >> (8 * (j % 4))) & 0xFFu));
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint32_t v  = d[4 * j + t];
                uint32_t lo = v & 0x0F0F0F0Fu, hi = (v >> 4) & 0x0F0F0F0Fu;
                /* (opaque, so that each byte is converted by one v_cvt_f32_ubyteN instead of
                 * being extracted from `v` again) */
                asm volatile("" : "+v"(lo), "+v"(hi));
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint32_t src = (i & 1) ? hi : lo;
                    const float    qf  = (float) ((src >> (8 * (i >> 1))) & 0xFFu);
                    const double   wv  = (double) __builtin_fmaf(d1, qf, nm1);
                    const int      k   = Q6K_BLOCK_ELEMS * b + 32 * j + 8 * t + i;
#pragma unroll
                    for (int m = 0; m < MT; ++m) {
                        const double *xm = xd + (long) (m < n_m ? m : n_m - 1) * n_in;
                        acc[m] = __builtin_fma(xm[k], wv, acc[m]); /* uniform address */
                    }
                }
            }
            if (j + 1 < 8) /* one sub-block at a time (see q6k_packed_half) */
                asm volatile("" : "+v"(acc[0]), "+v"(d[4 * j + 4]), "+v"(d[4 * j + 5]),
                                  "+v"(d[4 * j + 6]), "+v"(d[4 * j + 7]));
        }
    }
    if (row < n_out) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
            if (m < n_m)
                y[m * ld_y + row] = (float) acc[m];
    }
}

size_t q4k_packed_bytes(long n_out, int n_in) {
    return (size_t) ((n_out + 63) / 64) * (size_t) (n_in / Q6K_BLOCK_ELEMS) * Q4K_PACK_DWORDS * 4;
}

void launch_q4k_pack(hipStream_t stream, const uint8_t *w_q4k, long n_out, int n_in,
                     void *packed) {
    const int  nb    = n_in / Q6K_BLOCK_ELEMS;
    const long items = (n_out + 63) / 64 * nb;
    k_q4k_pack<<<dim3((unsigned) ((items + 3) / 4)), dim3(Q6K_TPB), 0, stream>>>(
        w_q4k, n_out, nb, static_cast<uint32_t *>(packed));
}

void launch_q4k_packed_linear(hipStream_t stream, const void *packed, long n_out, int n_in,
                              const float *x, long ld_x, int n_m, const Q6KScratch &ws, float *y,
                              long ld_y) {
    k_q6k_x_prep<<<dim3(n_m), dim3(Q6K_TPB), 0, stream>>>(x, ld_x, n_in, ws.xd, ws.xsum, ws.xabs,
                                                         ws.amb_count);
    const long     groups = (n_out + 63) / 64;
    const dim3     grid((unsigned) ((groups + 3) / 4)), block(Q6K_TPB);
    const uint32_t *p = static_cast<const uint32_t *>(packed);
    switch (n_m) {
    case 1: k_q4k_packed_linear<1><<<grid, block, 0, stream>>>(p, n_out, n_in, ws.xd, n_m, y, ld_y); break;
    case 2: k_q4k_packed_linear<2><<<grid, block, 0, stream>>>(p, n_out, n_in, ws.xd, n_m, y, ld_y); break;
    default: k_q4k_packed_linear<4><<<grid, block, 0, stream>>>(p, n_out, n_in, ws.xd, n_m, y, ld_y); break;
    }
}

} // namespace gs
