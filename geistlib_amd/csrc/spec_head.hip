/*
 * spec_head.hip -- the reference's speculative output head for greedy decoding
 * (src/archs/transformer/forward/spec_head.c) over a tied F16 table in device memory, for gfx950.
 *
 * Built once per model (spec_head.c:402-607): the `sketch_dim` dimensions of the table with the
 * largest variance over a sample of rows, every row's values in those dimensions as int8 with
 * one scale per row, and two norms per row for the certainty bound.
 *
 * Per token (spec_head.c:624-889):
 *   k_spec_act        the hidden row in int8, its kept dimensions, the activation norms
 *   k_q8w_gemv        rough[r] = (float)(a . sketch[r]) * row_scale[r]: the int8 projection kernel
 *                     of the dense head. The dot is formed in binary32 there, which is exact for
 *                     sums below 2^24 (sketch_dim <= 1040), so the scores equal the reference's
 *                     integer dot bit for bit. Its epilogue leaves the maxima of groups of 32
 *                     scores (the sampler's thread maxima).
 *   k_spec_threshold  the topk-th largest of those maxima: at least topk scores reach it, so
 *                     the topk best rows are among the rows >= it (about 1.1 topk rows)
 *   k_spec_gather     finds those rows and computes their exact logits, one wavefront per row,
 *                     in the order of summation of f16_gemv_m1 (16 chains, fixed tree), so that
 *                     a finalist's logit is the dense head's in every bit
 *   k_spec_final      the topk best rough scores among the listed rows (the reference's heap),
 *                     the best exact logit among them, lowest index first
 *   k_spec_verify     (optional, GEIST_SPEC_VERIFY) the upper bound of every excluded row
 *                     against the winner; any row that could have won withdraws the answer
 *
 * Differences from the reference that cannot show in a token: sums that only feed the bound
 * (norms of rows and of the activation) are accumulated in double here and in index order in
 * binary32 there. One that can: among rough scores equal to the topk-th best the reference keeps
 * whichever rows its heap's sift order leaves, this code the lowest indices.
 */
#include "spec_head_kernels.h"

#include "lm_head_kernels.h"

#include <hip/hip_fp16.h>

namespace gs {

namespace {

constexpr int SP_TPB  = 256;
constexpr int SP_WAVE = 64;

typedef uint32_t nt_u4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float h2f(uint16_t h) {
    return __half2float(__ushort_as_half(h));
}

/* Keys that order like the floats; NaN (an empty thread's maximum) sorts below everything. */
__device__ __forceinline__ uint32_t ordered_key(float f) {
    if (f != f)
        return 0u;
    const uint32_t b = __float_as_uint(f + 0.0f); /* -0 orders as +0 */
    return (b >> 31) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float key_to_float(uint32_t k) {
    return __uint_as_float((k >> 31) ? (k & 0x7fffffffu) : ~k);
}

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1)
        v += __shfl_xor(v, d, SP_WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1)
        v = __builtin_fmaxf(v, __shfl_xor(v, d, SP_WAVE));
    return v;
}

/* Inclusive scan over the 256 threads of a workgroup; s_w[4] is scratch. */
__device__ __forceinline__ int block_incl_scan(int v, int *s_w) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    int       x    = v;
#pragma unroll
    for (int d = 1; d < SP_WAVE; d <<= 1) {
        const int y = __shfl_up(x, d, SP_WAVE);
        if (lane >= d)
            x += y;
    }
    if (lane == 63)
        s_w[wv] = x;
    __syncthreads();
    int add = 0;
    for (int i = 0; i < wv; ++i)
        add += s_w[i];
    __syncthreads();
    return x + add;
}

/* The k-th largest (1 <= k <= n) of the n keys key_at(i), by four 8-bit radix passes of the
 * whole workgroup; need_ties = how many of the keys equal to it belong to the k largest. */
template <typename KeyAt>
__device__ uint32_t block_kth_largest(KeyAt key_at, int n, int k, int *s_hist, int *s_w, int *s_sel,
                                      int &need_ties) {
    const int tid    = threadIdx.x;
    uint32_t  prefix = 0, mask = 0;
    int       remaining = k;
    for (int shift = 24; shift >= 0; shift -= 8) {
        s_hist[tid] = 0;
        __syncthreads();
        for (int i = tid; i < n; i += SP_TPB) {
            const uint32_t key = key_at(i);
            if ((key & mask) == prefix)
                atomicAdd(&s_hist[(key >> shift) & 255u], 1);
        }
        __syncthreads();
        const int mine = s_hist[255 - tid]; /* thread t owns digit 255 - t: descending order */
        const int incl = block_incl_scan(mine, s_w);
        if (incl >= remaining && incl - mine < remaining) {
            s_sel[0] = 255 - tid;
            s_sel[1] = remaining - (incl - mine);
        }
        __syncthreads();
        prefix |= (uint32_t) s_sel[0] << shift;
        mask |= 255u << shift;
        remaining = s_sel[1];
        __syncthreads();
    }
    need_ties = remaining;
    return prefix;
}

/* ---- build ------------------------------------------------------------------------------- */

__global__ __launch_bounds__(SP_TPB) void k_spec_dim_stats(const uint16_t *__restrict__ w,
                                                           long vocab, int d_model, long vstep,
                                                           float *__restrict__ dvar) {
    const int i = blockIdx.x * SP_TPB + threadIdx.x;
    if (i >= d_model)
        return;
    float sum = 0.0f, sq = 0.0f;
    long  vn  = 0;
    for (long r = 0; r < vocab; r += vstep, ++vn) {
        const float v = h2f(w[r * d_model + i]);
        sum           = __fadd_rn(sum, v);
        sq            = __fadd_rn(sq, __fmul_rn(v, v));
    }
    const float mean = __fdiv_rn(sum, (float) vn);
    dvar[i]          = __fsub_rn(__fdiv_rn(sq, (float) vn), __fmul_rn(mean, mean));
}

/* One wavefront per table row. */
__global__ __launch_bounds__(SP_TPB) void k_spec_sketch_rows(SpecHeadDev d) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    uint16_t *row  = reinterpret_cast<uint16_t *>(smem) + (size_t) wv * d.d_model;
    const long r   = (long) blockIdx.x * (SP_TPB / SP_WAVE) + wv;
    if (r >= d.vocab)
        return; /* (no workgroup barrier below) */
    const uint16_t *src = d.w + r * d.d_model;
    for (int o = lane * 8; o < d.d_model; o += SP_WAVE * 8)
        *reinterpret_cast<uint4 *>(row + o) = *reinterpret_cast<const uint4 *>(src + o);
    /* largest magnitude over the kept dimensions (spec_head.c:571-578) */
    float amax = 0.0f;
    for (int s = lane; s < d.sketch_dim; s += SP_WAVE)
        amax = __builtin_fmaxf(amax, __builtin_fabsf(h2f(row[d.dims[s]])));
    amax = __builtin_fmaxf(wave_max(amax), 1e-8f);
    const float scale = __fdiv_rn(127.0f, amax);
    int8_t     *sk    = d.sketch + r * d.sketch_dim;
    for (int s = lane; s < d.sketch_dim; s += SP_WAVE) {
        float q = __builtin_rintf(__fmul_rn(h2f(row[d.dims[s]]), scale));
        q       = __builtin_fminf(__builtin_fmaxf(q, -127.0f), 127.0f);
        sk[s]   = (int8_t) (int) q;
    }
    /* norms for the bound (spec_head.c:591-602) */
    double l1 = 0.0, sq = 0.0;
    for (int i = lane; i < d.d_model; i += SP_WAVE) {
        const double v = (double) h2f(row[i]);
        if (d.kept[i])
            l1 += fabs(v);
        else
            sq += v * v;
    }
    l1 = wave_sum(l1);
    sq = wave_sum(sq);
    if (lane == 0) {
        d.row_scale[r] = __fdiv_rn(amax, 127.0f);
        d.w_drop[r]    = (float) sqrt(sq);
        d.w_l1[r]      = (float) l1;
    }
}

/* ---- per token --------------------------------------------------------------------------- */

/* spec_head.c:672-694 and 712-724, one workgroup. */
__global__ __launch_bounds__(SP_TPB) void k_spec_act(SpecHeadDev d, const float *__restrict__ h) {
    __shared__ float  s_max[SP_TPB / SP_WAVE];
    __shared__ double s_sum[3][SP_TPB / SP_WAVE];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    float     amax = 0.0f;
    double    all2 = 0.0;
    for (int i = tid; i < d.d_model; i += SP_TPB) {
        const float v = h[i];
        amax          = __builtin_fmaxf(amax, __builtin_fabsf(v));
        all2 += (double) v * (double) v;
    }
    amax = wave_max(amax);
    if (lane == 0)
        s_max[wv] = amax;
    __syncthreads();
    amax = 1e-8f;
    for (int i = 0; i < SP_TPB / SP_WAVE; ++i)
        amax = __builtin_fmaxf(amax, s_max[i]);
    const float x_q = __fdiv_rn(127.0f, amax);
    double      l1 = 0.0, kept2 = 0.0;
    for (int s = tid; s < d.sketch_dim; s += SP_TPB) {
        const float v = h[d.dims[s]];
        float       q = __builtin_rintf(__fmul_rn(v, x_q));
        q             = __builtin_fminf(__builtin_fmaxf(q, -127.0f), 127.0f);
        d.act[s]      = q;
        l1 += fabs((double) v);
        kept2 += (double) v * (double) v;
    }
    all2  = wave_sum(all2);
    l1    = wave_sum(l1);
    kept2 = wave_sum(kept2);
    if (lane == 0)
        s_sum[0][wv] = all2, s_sum[1][wv] = l1, s_sum[2][wv] = kept2;
    __syncthreads();
    if (tid == 0) {
        double a = 0.0, b = 0.0, c = 0.0;
        for (int i = 0; i < SP_TPB / SP_WAVE; ++i)
            a += s_sum[0][i], b += s_sum[1][i], c += s_sum[2][i];
        const double drop = a - c > 0.0 ? a - c : 0.0;
        d.sc->inv_xq      = __fdiv_rn(1.0f, x_q);
        d.sc->h_l1_kept   = (float) b;
        d.sc->h_l2_drop   = (float) sqrt(drop);
        d.sc->n_listed    = 0;
    }
}

__global__ __launch_bounds__(SP_TPB) void k_spec_threshold(SpecHeadDev d) {
    __shared__ int s_hist[256], s_w[4], s_sel[2];
    const float   *tm = d.tmax;
    int            ties;
    const uint32_t key = block_kth_largest([tm](int i) { return ordered_key(tm[i]); },
                                           d.n_chunks * 256, d.topk, s_hist, s_w, s_sel, ties);
    if (threadIdx.x == 0)
        d.sc->threshold = key_to_float(key);
}

/* Rows whose rough score reaches the threshold, and their exact logits. Thread t of workgroup b
 * looks at row 256 b + t; every such row is then worked on by its whole wavefront: the row comes
 * into LDS with coalesced 16-byte loads, lanes 0..15 each run one of f16_gemv_m1's sixteen
 * chains over it (element k belongs to chain k % 16; a trailing block of eight extends chains
 * 0..7), and the chains are folded as there: (j + j+8), (i + i+4), ((0+1) + (2+3))
 * (src/backends/cpu_x86/kernel_f16_gemv.c:25-32, 40-59). */
__global__ __launch_bounds__(SP_TPB) void k_spec_gather(SpecHeadDev d, const float *__restrict__ h) {
    extern __shared__ __align__(16) uint8_t smem[];
    float    *s_x   = reinterpret_cast<float *>(smem);
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    uint16_t *s_row = reinterpret_cast<uint16_t *>(smem + (size_t) d.d_model * 4) +
                      (size_t) wv * d.d_model;
    const long  r   = (long) blockIdx.x * SP_TPB + tid;
    const float thr = d.sc->threshold;
    const float val = r < d.vocab ? d.rough[r] : -__builtin_inff();
    const bool  hit = r < d.vocab && val >= thr;
    if (__syncthreads_or(hit) == 0)
        return;
    for (int i = tid * 4; i < d.d_model; i += SP_TPB * 4)
        *reinterpret_cast<float4 *>(s_x + i) = *reinterpret_cast<const float4 *>(h + i);
    __syncthreads();
    unsigned long long mask = __ballot(hit);
    const int          n16  = d.d_model & ~15;
    while (mask) {
        const int  bit = __builtin_ctzll(mask);
        mask &= mask - 1;
        const long cr  = (long) blockIdx.x * SP_TPB + wv * SP_WAVE + bit;
        const uint16_t *src = d.w + cr * d.d_model;
        for (int o = lane * 8; o < d.d_model; o += SP_WAVE * 8)
            *reinterpret_cast<nt_u4 *>(s_row + o) =
                __builtin_nontemporal_load(reinterpret_cast<const nt_u4 *>(src + o));
        float acc = 0.0f;
        if (lane < 16) {
            for (int k = lane; k < n16; k += 16)
                acc = __builtin_fmaf(h2f(s_row[k]), s_x[k], acc);
            if ((d.d_model & 15) == 8 && lane < 8)
                acc = __builtin_fmaf(h2f(s_row[n16 + lane]), s_x[n16 + lane], acc);
        }
        const float v   = __fadd_rn(acc, __shfl_down(acc, 8, SP_WAVE));
        const float q   = __fadd_rn(v, __shfl_down(v, 4, SP_WAVE));
        const float a   = __fadd_rn(q, __shfl_down(q, 1, SP_WAVE));
        const float sum = __fadd_rn(a, __shfl_down(a, 2, SP_WAVE));
        const float rv  = __shfl(val, bit, SP_WAVE);
        if (lane == 0) {
            const int slot = atomicAdd(&d.sc->n_listed, 1);
            if (slot < d.list_cap) {
                d.list_idx[slot]   = (int32_t) cr;
                d.list_rough[slot] = rv;
                d.list_exact[slot] = sum;
            }
        }
    }
}

/* The topk best rough scores among the listed rows and the best exact logit among those
 * (spec_head.c:728-770, 802-827), one workgroup. */
__global__ __launch_bounds__(SP_TPB) void k_spec_final(SpecHeadDev d, SpecResult *__restrict__ res) {
    __shared__ int      s_hist[256], s_w[4], s_sel[2];
    __shared__ uint64_t s_best[SP_TPB / SP_WAVE];
    __shared__ int      s_cnt[SP_TPB / SP_WAVE];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int listed = d.sc->n_listed;
    if (listed > d.list_cap || listed < d.topk) { /* (uniform) more equal scores than the list holds */
        if (tid == 0) {
            res->token = -1, res->answered = 0, res->n_finalists = 0, res->n_listed = listed;
            res->cutoff = d.sc->threshold, res->best_exact = 0.0f;
        }
        return;
    }
    const float *lr = d.list_rough;
    int          need_ties;
    const uint32_t ckey = block_kth_largest([lr](int i) { return ordered_key(lr[i]); }, listed,
                                            d.topk, s_hist, s_w, s_sel, need_ties);
    uint64_t best = 0;
    int      cnt  = 0;
    for (int i = tid; i < listed; i += SP_TPB) {
        const uint32_t key = ordered_key(lr[i]);
        bool           in  = key > ckey;
        if (key == ckey) { /* the lowest indices among the rows that tie at the cutoff */
            const int32_t me = d.list_idx[i];
            int           before = 0;
            for (int j = 0; j < listed; ++j)
                before += (ordered_key(lr[j]) == ckey && d.list_idx[j] < me) ? 1 : 0;
            in = before < need_ties;
        }
        if (in) {
            ++cnt;
            const uint64_t p = ((uint64_t) ordered_key(d.list_exact[i]) << 32) |
                               (uint32_t) (0x7fffffff - d.list_idx[i]);
            best = p > best ? p : best;
        }
    }
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) {
        const uint64_t o = __shfl_xor(best, s, SP_WAVE);
        best             = o > best ? o : best;
        cnt += __shfl_xor(cnt, s, SP_WAVE);
    }
    if (lane == 0)
        s_best[wv] = best, s_cnt[wv] = cnt;
    __syncthreads();
    if (tid == 0) {
        for (int i = 1; i < SP_TPB / SP_WAVE; ++i) {
            best = s_best[i] > best ? s_best[i] : best;
            cnt += s_cnt[i];
        }
        res->token       = 0x7fffffff - (int32_t) (uint32_t) (best & 0xffffffffu);
        res->answered    = 1;
        res->n_finalists = cnt;
        res->n_listed    = listed;
        res->cutoff      = key_to_float(ckey);
        res->best_exact  = key_to_float((uint32_t) (best >> 32));
    }
}

/* spec_head.c:846-872: a row outside the finalists whose upper bound passes the winner's exact
 * logit withdraws the answer. */
__global__ __launch_bounds__(SP_TPB) void k_spec_verify(SpecHeadDev d, SpecResult *__restrict__ res) {
    const long r = (long) blockIdx.x * SP_TPB + threadIdx.x;
    if (r >= d.vocab || res->n_finalists == 0)
        return;
    const float rough = d.rough[r];
    if (rough > res->cutoff)
        return;
    const float inv_xq = d.sc->inv_xq;
    float ub = __fmul_rn(rough, inv_xq);
    ub = __fadd_rn(ub, __fmul_rn(__fmul_rn(0.5f, d.row_scale[r]), d.sc->h_l1_kept));
    ub = __fadd_rn(ub, __fmul_rn(__fmul_rn(0.5f, d.w_l1[r]), inv_xq));
    ub = __fadd_rn(ub, __fmul_rn(d.w_drop[r], d.sc->h_l2_drop));
    if (ub > res->best_exact)
        res->answered = 0;
}

} // namespace

void launch_spec_dim_stats(hipStream_t stream, const uint16_t *w, long vocab, int d_model,
                           long vstep, float *dvar) {
    k_spec_dim_stats<<<dim3((unsigned) ((d_model + SP_TPB - 1) / SP_TPB)), dim3(SP_TPB), 0, stream>>>(
        w, vocab, d_model, vstep, dvar);
}

void launch_spec_sketch_rows(hipStream_t stream, const SpecHeadDev &d) {
    const int    rows_block = SP_TPB / SP_WAVE;
    const size_t lds        = (size_t) rows_block * d.d_model * sizeof(uint16_t);
    k_spec_sketch_rows<<<dim3((unsigned) ((d.vocab + rows_block - 1) / rows_block)), dim3(SP_TPB), lds,
                         stream>>>(d);
}

void launch_spec_try(hipStream_t stream, const SpecHeadDev &d, const float *h, bool verify,
                     SpecResult *result) {
    const dim3 one(1), block(SP_TPB), rows((unsigned) ((d.vocab + SP_TPB - 1) / SP_TPB));
    k_spec_act<<<one, block, 0, stream>>>(d, h);
    GemvFuse f{};
    f.tmax     = d.tmax;
    f.n_chunks = d.n_chunks;
    launch_q8w_gemv(stream, d.sketch, d.row_scale, d.vocab, d.sketch_dim, d.act, d.sketch_dim, 1,
                    d.rough, d.vocab, &f);
    k_spec_threshold<<<one, block, 0, stream>>>(d);
    const size_t lds = (size_t) d.d_model * (sizeof(float) + (SP_TPB / SP_WAVE) * sizeof(uint16_t));
    k_spec_gather<<<rows, block, lds, stream>>>(d, h);
    k_spec_final<<<one, block, 0, stream>>>(d, result);
    if (verify)
        k_spec_verify<<<rows, block, 0, stream>>>(d, result);
}

} // namespace gs
