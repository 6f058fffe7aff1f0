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
 *                     integer dot bit for bit. Its epilogue leaves the maximum of every group
 *                     of 32 consecutive scores (the rows one wavefront computes).
 *   k_spec_select     the topk-th largest of those maxima: at least topk scores reach it, so
 *                     the topk best rows are among the rows >= it (about 1.1 topk rows); it
 *                     reads those groups again and keeps the topk best (the reference's heap)
 *   k_spec_exact      their exact logits, one wavefront per row, in the order of summation of
 *                     f16_gemv_m1 (16 chains, fixed tree), so that a finalist's logit is the
 *                     dense head's in every bit
 *   k_spec_final      the best exact logit among them, lowest index first
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
#include "rmsnorm_device.h"

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

/* One count for this lane's digit (if valid). Keys that order like floats share their leading
 * digits, and atomics of one wavefront on one LDS word are serialised: the lanes that hold the
 * digit of the first valid lane add their count in one operation, the others one by one. */
__device__ __forceinline__ void hist_add(int *s_hist, uint32_t digit, bool valid) {
    const unsigned long long todo = __ballot(valid);
    if (todo == 0)
        return;
    const int                leader = __builtin_ctzll(todo);
    const uint32_t           dl = (uint32_t) __builtin_amdgcn_readlane((int) digit, leader);
    const unsigned long long m  = __ballot(valid && digit == dl);
    if ((int) (threadIdx.x & 63) == leader)
        atomicAdd(&s_hist[dl], __builtin_popcountll(m));
    if (valid && digit != dl)
        atomicAdd(&s_hist[digit], 1);
}

/* The k-th largest (1 <= k <= n) of the keys the workgroup's threads hold in registers (thread t
 * holds keys[e] for the elements e * blockDim.x + t < n), by four 8-bit radix passes;
 * need_ties = how many of the keys equal to it belong to the k largest. s_hist is [4][256].
 * With PASSES < 4 only the leading 8 * PASSES bits are resolved: the result is the k-th largest
 * key with its other bits cleared (a lower bound of it that at least k keys reach).
 * Each pass costs two workgroup barriers: all wavefronts count their digits, then the first
 * wavefront alone finds the digit that holds the k-th key (lane l owns the digits 255 - 4 l ..
 * 252 - 4 l, so that a scan over the lanes runs from the largest digit down). */
template <int EPT, int PASSES = 4>
__device__ uint32_t block_kth_largest(const uint32_t (&keys)[EPT], int n, int k, int (*s_hist)[256],
                                      int *s_sel, int &need_ties) {
    const int tid = threadIdx.x, lane = tid & 63;
    for (int i = tid; i < 4 * 256; i += (int) blockDim.x)
        (&s_hist[0][0])[i] = 0;
    __syncthreads();
    uint32_t prefix = 0, mask = 0;
    int      remaining = k;
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
        const int shift = 24 - 8 * pass;
#pragma unroll
        for (int e = 0; e < EPT; ++e)
            hist_add(s_hist[pass], (keys[e] >> shift) & 255u,
                     e * (int) blockDim.x + tid < n && (keys[e] & mask) == prefix);
        __syncthreads();
        if (tid < SP_WAVE) {
            int c[4], local = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                c[j] = s_hist[pass][255 - 4 * lane - j];
                local += c[j];
            }
            int incl = local;
#pragma unroll
            for (int d = 1; d < SP_WAVE; d <<= 1) {
                const int y = __shfl_up(incl, d, SP_WAVE);
                if (lane >= d)
                    incl += y;
            }
            int r = remaining - (incl - local);
            if (r >= 1 && r <= local) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (r >= 1 && r <= c[j]) {
                        s_sel[0] = 255 - 4 * lane - j;
                        s_sel[1] = r;
                    }
                    r -= c[j];
                }
            }
        }
        __syncthreads();
        prefix |= (uint32_t) s_sel[0] << shift;
        mask |= 255u << shift;
        remaining = s_sel[1];
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

/* spec_head.c:672-694 and 712-724, one workgroup. With NORM the output norm of head.c:99-101
 * runs in front: h = (x * inv_rms) * norm_w, written to h_out for the finalist kernel, in the
 * arithmetic of the norm kernel of the dense head. */
template <bool NORM>
__global__ __launch_bounds__(SP_TPB) void k_spec_act(SpecHeadDev d, const float *__restrict__ h_in,
                                                     const float *__restrict__ norm_w, float eps,
                                                     float *__restrict__ h_out) {
    __shared__ float  s_max[SP_TPB / SP_WAVE];
    __shared__ double s_sum[3][SP_TPB / SP_WAVE];
    __shared__ double s_part[NORM ? SP_TPB : 1];
    __shared__ float  s_inv;
    __shared__ float  s_h[NORM ? SPEC_D_MODEL_MAX : 1];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const float *h = h_in;
    if (NORM) {
        const float inv = block_rms_inv<SP_TPB>(h_in, d.d_model, eps, s_part, &s_inv);
        for (int i = tid; i < d.d_model; i += SP_TPB) {
            const float y = __fmul_rn(__fmul_rn(h_in[i], inv), norm_w[i]);
            s_h[i]        = y;
            h_out[i]      = y;
        }
        __syncthreads();
        h = s_h;
    }
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
    }
}

constexpr int SP_SEL_TPB = 1024; /* the two selection kernels: keys live in registers */

/* Phase 2 of the head (spec_head.c:728-770), one workgroup of 1024 threads:
 *   1. the topk-th largest group maximum (group g = rows 32 g .. 32 g + 31, written by the
 *      projection's epilogue), to 16 bits: at least topk rough scores reach it, so the topk
 *      best rows are among the rows >= it;
 *   2. only the groups whose maximum reaches that threshold are read again, their rows >= it
 *      are the candidates (about 1.1 topk, at most 2 topk);
 *   3. the topk-th largest candidate is the reference's cutoff (its heap's smallest entry); the
 *      finalists are the candidates above it and, of those equal to it, as many as complete
 *      topk rows -- the lowest indices first.
 * Thread t holds the maxima e * 1024 + t and later the candidates e * 1024 + t. */
template <int EPT, int EPT2, int IT>
__global__ __launch_bounds__(SP_SEL_TPB) void k_spec_select(SpecHeadDev d) {
    extern __shared__ __align__(16) uint8_t smem[];
    int      *s_ent = reinterpret_cast<int *>(smem); /* [list_cap] groups to read again */
    int32_t  *s_ci  = s_ent + d.list_cap;             /* [list_cap] candidate rows */
    uint32_t *s_ck  = reinterpret_cast<uint32_t *>(s_ci + d.list_cap); /* ... and their keys */
    __shared__ int s_hist[4][256], s_w[16], s_sel[2], s_n[3];
    const int tid = threadIdx.x, lane = tid & 63;
    const int n   = d.n_groups;
    uint32_t  keys[EPT];
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
        const int i = e * SP_SEL_TPB + tid;
        keys[e]     = i < n ? ordered_key(d.gmax[i]) : 0u;
    }
    if (tid < 3)
        s_n[tid] = 0;
    /* (16 bits of the threshold are enough: it only has to be reached by at least topk maxima
     * and by few more rows than topk; the exact cutoff comes from the candidates below) */
    int            ties;
    const uint32_t tkey = block_kth_largest<EPT, 2>(keys, n, d.topk, s_hist, s_sel, ties);
    const float    thr  = key_to_float(tkey);
    /* 2a. the groups that reach the threshold */
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
        const int  i   = e * SP_SEL_TPB + tid;
        const bool hit = i < n && keys[e] >= tkey && keys[e] != 0u;
        const unsigned long long m = __ballot(hit);
        if (m == 0)
            continue;
        int base = 0;
        if (lane == 0)
            base = atomicAdd(&s_n[0], __builtin_popcountll(m));
        base = __builtin_amdgcn_readfirstlane(base);
        const int slot = base + __builtin_popcountll(m & ((1ull << lane) - 1ull));
        if (hit && slot < d.list_cap)
            s_ent[slot] = i;
    }
    __syncthreads();
    const int n_ent = s_n[0] < d.list_cap ? s_n[0] : d.list_cap;
    /* 2b. their rows that reach it, into the candidate list in LDS: IT groups per thread and
     * round with all their loads in flight together. A wavefront counts its hits with one ballot
     * per row position, takes its slots with one atomic and hands them out by ballot again
     * (candidates are stored in no particular order). */
    for (int round = 0; round < n_ent; round += IT * SP_SEL_TPB) { /* (uniform) */
        float v[IT][32];
        long  base[IT];
#pragma unroll
        for (int u = 0; u < IT; ++u) {
            const int  it   = round + u * SP_SEL_TPB + tid;
            const bool live = it < n_ent;
            const int  i    = live ? s_ent[it] : 0;
            base[u]         = (long) i * 32;
            /* (no branch around a load, so that all of them are in flight together: rough is
             * allocated in whole groups, rows beyond the vocabulary are masked afterwards) */
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const long   r0 = base[u] + 4 * j;
                const float4 f  = *reinterpret_cast<const float4 *>(d.rough + r0);
                v[u][4 * j]     = live && r0 + 0 < d.vocab ? f.x : -__builtin_inff();
                v[u][4 * j + 1] = live && r0 + 1 < d.vocab ? f.y : -__builtin_inff();
                v[u][4 * j + 2] = live && r0 + 2 < d.vocab ? f.z : -__builtin_inff();
                v[u][4 * j + 3] = live && r0 + 3 < d.vocab ? f.w : -__builtin_inff();
            }
        }
#pragma unroll
        for (int u = 0; u < IT; ++u) {
            if (round + u * SP_SEL_TPB + tid - lane >= n_ent)
                continue; /* (whole wavefronts) */
            int total = 0;
#pragma unroll
            for (int j = 0; j < 32; ++j)
                total += __builtin_popcountll(__ballot(v[u][j] >= thr));
            int wbase = 0;
            if (lane == 0)
                wbase = atomicAdd(&s_n[1], total);
            wbase = __builtin_amdgcn_readfirstlane(wbase);
#pragma unroll
            for (int j = 0; j < 32; ++j) {
                const bool               hit = v[u][j] >= thr;
                const unsigned long long m   = __ballot(hit);
                const int slot = wbase + __builtin_popcountll(m & ((1ull << lane) - 1ull));
                if (hit && slot < d.list_cap) {
                    s_ci[slot] = (int32_t) (base[u] + j);
                    s_ck[slot] = ordered_key(v[u][j]);
                }
                wbase += __builtin_popcountll(m);
            }
        }
    }
    __syncthreads();
    const int n_cand = s_n[1];
    if (s_n[0] > d.list_cap || n_cand > d.list_cap || n_cand < d.topk) { /* (uniform) */
        if (tid == 0) {
            d.sc->threshold = thr, d.sc->cutoff = thr, d.sc->n_cand = n_cand, d.sc->n_final = 0;
        }
        return;
    }
    /* 3. the cutoff and the finalists */
    uint32_t ck[EPT2];
    int32_t  ci[EPT2];
#pragma unroll
    for (int e = 0; e < EPT2; ++e) {
        const int i = e * SP_SEL_TPB + tid;
        ck[e]       = i < n_cand ? s_ck[i] : 0u;
        ci[e]       = i < n_cand ? s_ci[i] : -1;
    }
    int            need_ties;
    const uint32_t ckey = block_kth_largest<EPT2>(ck, n_cand, d.topk, s_hist, s_sel, need_ties);
    int tie_cnt = 0;
#pragma unroll
    for (int e = 0; e < EPT2; ++e)
        tie_cnt += (ci[e] >= 0 && ck[e] == ckey) ? 1 : 0;
#pragma unroll
    for (int sft = 32; sft >= 1; sft >>= 1)
        tie_cnt += __shfl_xor(tie_cnt, sft, SP_WAVE);
    if (lane == 0)
        s_w[tid >> 6] = tie_cnt;
    __syncthreads();
    tie_cnt = 0;
    for (int i = 0; i < SP_SEL_TPB / SP_WAVE; ++i)
        tie_cnt += s_w[i];
#pragma unroll
    for (int e = 0; e < EPT2; ++e) {
        bool in = ci[e] >= 0 && ck[e] > ckey;
        if (ci[e] >= 0 && ck[e] == ckey) {
            in = true;
            if (tie_cnt > need_ties) { /* the lowest indices among the rows that tie */
                int before = 0;
                for (int j = 0; j < n_cand; ++j)
                    before += (s_ci[j] < ci[e] && s_ck[j] == ckey) ? 1 : 0;
                in = before < need_ties;
            }
        }
        const unsigned long long m = __ballot(in);
        if (m == 0)
            continue;
        int base = 0;
        if (lane == 0)
            base = atomicAdd(&s_n[2], __builtin_popcountll(m));
        base = __builtin_amdgcn_readfirstlane(base);
        const int slot = base + __builtin_popcountll(m & ((1ull << lane) - 1ull));
        if (in && slot < d.topk)
            d.fin_idx[slot] = ci[e];
    }
    __syncthreads();
    if (tid == 0) {
        d.sc->threshold = thr;
        d.sc->cutoff    = key_to_float(ckey);
        d.sc->n_cand    = n_cand;
        d.sc->n_final   = s_n[2]; /* == topk */
    }
}

/* Phase 3 (spec_head.c:802-826): the exact logit of every finalist, one wavefront per row, in
 * f16_gemv_m1's order of summation (src/backends/cpu_x86/kernel_f16_gemv.c:25-32, 40-59):
 * sixteen chains of fused multiply-adds, element k in chain k % 16, folded as (j + j+8),
 * (i + i+4), ((0+1) + (2+3)). Lane c < 16 runs chain c. Row and activations are laid out in LDS
 * by chain (element k at (k % 16) * pitch + k / 16), so that a lane reads its chain's next
 * eight weights with one 16-byte load. d_model is a multiple of 16. */
__global__ __launch_bounds__(SP_TPB) void k_spec_exact(SpecHeadDev d, const float *__restrict__ h) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int per   = d.d_model >> 4;     /* elements per chain */
    const int pitch = (per + 7) & ~7;
    float    *s_x   = reinterpret_cast<float *>(smem);                       /* [16][pitch] */
    uint16_t *s_row = reinterpret_cast<uint16_t *>(smem + (size_t) 16 * pitch * 4) +
                      (size_t) wv * 16 * pitch;                              /* [16][pitch] */
    const int n_final = d.sc->n_final;
    if ((int) blockIdx.x * (SP_TPB / SP_WAVE) >= n_final)
        return; /* (uniform) */
    /* the activations are requested first and stored last, so that their latency and the row's
     * overlap */
    constexpr int X_PER_THREAD = SPEC_D_MODEL_MAX / SP_TPB;
    float         xv[X_PER_THREAD];
#pragma unroll
    for (int i = 0; i < X_PER_THREAD; ++i)
        xv[i] = i * SP_TPB + tid < d.d_model ? h[i * SP_TPB + tid] : 0.0f;
    const int slot = (int) blockIdx.x * (SP_TPB / SP_WAVE) + wv;
    if (slot < n_final) {
        const uint16_t *src = d.w + (long) d.fin_idx[slot] * d.d_model;
        for (int o = lane * 8; o < d.d_model; o += SP_WAVE * 8) {
            const nt_u4 q = __builtin_nontemporal_load(reinterpret_cast<const nt_u4 *>(src + o));
            /* elements o .. o+7: chains (o & 15) .. (o & 15) + 7 at position o / 16 */
            uint16_t *dst = s_row + (o & 15) * pitch + (o >> 4);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                dst[(2 * i) * pitch]     = (uint16_t) (q[i] & 0xffffu);
                dst[(2 * i + 1) * pitch] = (uint16_t) (q[i] >> 16);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < X_PER_THREAD; ++i) {
        const int k = i * SP_TPB + tid;
        if (k < d.d_model)
            s_x[(k & 15) * pitch + (k >> 4)] = xv[i];
    }
    __syncthreads();
    if (slot >= n_final)
        return; /* (no workgroup barrier below) */
    float acc = 0.0f;
    if (lane < 16) {
        const uint16_t *wr = s_row + lane * pitch;
        const float    *xr = s_x + lane * pitch;
        int             p  = 0;
        for (; p + 8 <= per; p += 8) {
            const uint4  q  = *reinterpret_cast<const uint4 *>(wr + p);
            const float4 xa = *reinterpret_cast<const float4 *>(xr + p);
            const float4 xb = *reinterpret_cast<const float4 *>(xr + p + 4);
            acc = __builtin_fmaf(h2f((uint16_t) (q.x & 0xffffu)), xa.x, acc);
            acc = __builtin_fmaf(h2f((uint16_t) (q.x >> 16)), xa.y, acc);
            acc = __builtin_fmaf(h2f((uint16_t) (q.y & 0xffffu)), xa.z, acc);
            acc = __builtin_fmaf(h2f((uint16_t) (q.y >> 16)), xa.w, acc);
            acc = __builtin_fmaf(h2f((uint16_t) (q.z & 0xffffu)), xb.x, acc);
            acc = __builtin_fmaf(h2f((uint16_t) (q.z >> 16)), xb.y, acc);
            acc = __builtin_fmaf(h2f((uint16_t) (q.w & 0xffffu)), xb.z, acc);
            acc = __builtin_fmaf(h2f((uint16_t) (q.w >> 16)), xb.w, acc);
        }
        for (; p < per; ++p)
            acc = __builtin_fmaf(h2f(wr[p]), xr[p], acc);
    }
    const float v   = __fadd_rn(acc, __shfl_down(acc, 8, SP_WAVE));
    const float q   = __fadd_rn(v, __shfl_down(v, 4, SP_WAVE));
    const float a   = __fadd_rn(q, __shfl_down(q, 1, SP_WAVE));
    const float sum = __fadd_rn(a, __shfl_down(a, 2, SP_WAVE));
    if (lane == 0)
        d.fin_exact[slot] = sum;
}

/* The best exact logit among the finalists, the lowest index among equals (spec_head.c:827),
 * one workgroup. */
__global__ __launch_bounds__(SP_SEL_TPB) void k_spec_final(SpecHeadDev d, SpecResult *__restrict__ res) {
    __shared__ uint64_t s_best[SP_SEL_TPB / SP_WAVE];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int n_final = d.sc->n_final;
    if (n_final == 0) { /* (uniform) more candidates around the cutoff than the list holds */
        if (tid == 0) {
            res->token = -1, res->answered = 0, res->n_finalists = 0, res->n_listed = d.sc->n_cand;
            res->cutoff = d.sc->cutoff, res->best_exact = 0.0f;
        }
        return;
    }
    uint64_t best = 0;
    for (int i = tid; i < n_final; i += SP_SEL_TPB) {
        const uint64_t p = ((uint64_t) ordered_key(d.fin_exact[i]) << 32) |
                           (uint32_t) (0x7fffffff - d.fin_idx[i]);
        best = p > best ? p : best;
    }
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) {
        const uint64_t o = __shfl_xor(best, s, SP_WAVE);
        best             = o > best ? o : best;
    }
    if (lane == 0)
        s_best[wv] = best;
    __syncthreads();
    if (tid == 0) {
        for (int i = 1; i < SP_SEL_TPB / SP_WAVE; ++i)
            best = s_best[i] > best ? s_best[i] : best;
        res->token       = 0x7fffffff - (int32_t) (uint32_t) (best & 0xffffffffu);
        res->answered    = 1;
        res->n_finalists = n_final;
        res->n_listed    = d.sc->n_cand;
        res->cutoff      = d.sc->cutoff;
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
                     SpecResult *result, const float *norm_w, float eps, float *h_normed) {
    const dim3 one(1), block(SP_TPB), sel(SP_SEL_TPB);
    const dim3 rows((unsigned) ((d.vocab + SP_TPB - 1) / SP_TPB));
    if (norm_w != nullptr) {
        k_spec_act<true><<<one, block, 0, stream>>>(d, h, norm_w, eps, h_normed);
        h = h_normed;
    } else {
        k_spec_act<false><<<one, block, 0, stream>>>(d, h, nullptr, 0.0f, nullptr);
    }
    GemvFuse f{};
    f.gmax = d.gmax;
    launch_q8w_gemv(stream, d.sketch, d.row_scale, d.vocab, d.sketch_dim, d.act, d.sketch_dim, 1,
                    d.rough, d.vocab, &f);
    /* group maxima: one per 32 rows; candidates: at most 2 topk */
    const size_t lds_sel = (size_t) d.list_cap * 3 * sizeof(int);
    if (d.n_groups <= 4 * SP_SEL_TPB && d.list_cap <= 2 * SP_SEL_TPB) {
        k_spec_select<4, 2, 2><<<one, sel, lds_sel, stream>>>(d);
    } else { /* up to 96 KB of LDS, above what a launch may take by default */
        if (d.n_groups <= 8 * SP_SEL_TPB) {
            (void) hipFuncSetAttribute(
                reinterpret_cast<const void *>(k_spec_select<8, SPEC_LIST_EPT_MAX, 1>),
                hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds_sel);
            k_spec_select<8, SPEC_LIST_EPT_MAX, 1><<<one, sel, lds_sel, stream>>>(d);
        } else {
            (void) hipFuncSetAttribute(
                reinterpret_cast<const void *>(
                    k_spec_select<SPEC_TMAX_EPT_MAX, SPEC_LIST_EPT_MAX, 1>),
                hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds_sel);
            k_spec_select<SPEC_TMAX_EPT_MAX, SPEC_LIST_EPT_MAX, 1><<<one, sel, lds_sel, stream>>>(d);
        }
    }
    const int    pitch = ((d.d_model >> 4) + 7) & ~7;
    const size_t lds   = (size_t) 16 * pitch * (sizeof(float) + (SP_TPB / SP_WAVE) * sizeof(uint16_t));
    k_spec_exact<<<dim3((unsigned) ((d.topk + 3) / 4)), block, lds, stream>>>(d, h);
    k_spec_final<<<one, sel, 0, stream>>>(d, result);
    if (verify)
        k_spec_verify<<<rows, block, 0, stream>>>(d, result);
}

} // namespace gs
