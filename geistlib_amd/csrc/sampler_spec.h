/*
 * sampler_spec.h -- speculative-decode verification (rejection sampling). Included by
 * sampler_kernels.hip. The reference has no counterpart: its speculative loop accepts by exact
 * match only (src/engine/session.c:599-606) and documents the missing rejection step
 * (include/geist_util.h:233-240). The batch shape is the reference's verify_forward: L+1
 * target rows per sequence (src/archs/transformer/arch_ops.c:176-270).
 *
 * Per sequence s with draft tokens x_0..x_{L-1}, draft probabilities q_j, target rows 0..L:
 *   p_j  = softmax of target row j as the reference forms it (sampler.c:68-85, 251-253);
 *   j*   = first j with not( u_j * q_j(x_j) < p_j(x_j) )   (exact: products of two floats in double);
 *   j* < L : token ~ max(0, p_j* - q_j*) / R, walked in index order with u_L;
 *   j* = L : token ~ p_L, the temperature sampler's walk (sampler.c:90-102) with u_L.
 *
 * Kernels (after k_tmax_scan + k_chunk_expsum over all n_seq * (L+1) target rows):
 *   k_spec_resid   grid (chunks, n_seq): finds j* and sums max(0, p - q) over its chunk of row j*
 *   k_spec_final   grid (n_seq): finds j* again, writes the accepted ids, draws the last token
 */
#ifndef GEIST_SAMPLER_SPEC_H
#define GEIST_SAMPLER_SPEC_H

namespace gs {

struct SpecArgs {
    int             L;       /* draft length */
    int             greedy;  /* T <= 0: exact match against the row argmax */
    float           inv_t;
    const float    *q;       /* [n_seq][L][n_vocab], row stride ld_q */
    long            ld_q;
    const int32_t  *draft;   /* [n_seq][L] */
    const float    *uniforms; /* [n_seq][L+1] */
    const uint64_t *chunk_best;
    const double   *chunk_sum;
    const float    *probe_p; /* unnormalised p_j(x_j) per target row */
    double         *resid_sum; /* [n_seq][chunks] */
    int32_t        *out_tokens; /* [n_seq][L+1] */
    int32_t        *n_accepted; /* [n_seq] */
};

constexpr int SPEC_L_MAX = 63;

struct SpecShared {
    double   row_sum[SPEC_L_MAX + 1];
    uint64_t row_best[SPEC_L_MAX + 1];
    float    q_tok[SPEC_L_MAX + 1];
    int      first_reject;
};

/* Sums of every target row of the sequence (chunk order), the row maxima, q_j(x_j), then the
 * first rejected position. Every thread returns j* (L when all drafts are accepted). */
__device__ __forceinline__ int spec_first_reject(const RowView &rv, const SpecArgs &a, int seq,
                                                 SpecShared &sh) {
    const int tid = threadIdx.x, C = rv.n_chunks, L = a.L;
    if (tid <= L) {
        const long row = (long) seq * (L + 1) + tid;
        uint64_t   b   = 0;
        for (int c = 0; c < C; ++c) {
            const uint64_t p = a.chunk_best[row * C + c];
            b                = p > b ? p : b;
        }
        sh.row_best[tid] = b;
        if (!a.greedy) {
            double tot = 0.0;
            for (int c = 0; c < C; ++c)
                tot += a.chunk_sum[row * C + c];
            sh.row_sum[tid] = tot;
            float qt        = 0.0f;
            if (tid < L) {
                const int x = a.draft[(long) seq * L + tid];
                if (x >= 0 && x < rv.n_vocab)
                    qt = a.q[((long) seq * L + tid) * a.ld_q + x];
            }
            sh.q_tok[tid] = qt;
        }
    }
    __syncthreads();
    if (tid == 0) {
        int j = 0;
        for (; j < L; ++j) {
            const long row = (long) seq * (L + 1) + j;
            const int  x   = a.draft[(long) seq * L + j];
            bool       ok;
            if (a.greedy) {
                /* a NaN at index 0 keeps the argmax at 0 (sampler.c:52-62) */
                const float first = rv.logits[row * rv.ld];
                const int   am    = (first != first) ? 0 : (int) best_idx(sh.row_best[j]);
                ok                = x == am;
            } else {
                float pn = 0.0f;
                if (x >= 0 && x < rv.n_vocab)
                    pn = (float) ((double) a.probe_p[row] / sh.row_sum[j]);
                ok = (double) a.uniforms[(long) seq * (L + 1) + j] * (double) sh.q_tok[j] <
                     (double) pn;
            }
            if (!ok)
                break;
        }
        sh.first_reject = j;
    }
    __syncthreads();
    return sh.first_reject;
}

/* The four weights thread `tid` owns in slab j of a chunk: p_i (temperature walk) or
 * max(0, pn_i - q_i) (residual walk). Positions at or beyond `end` weigh 0. */
template <bool RESID>
__device__ __forceinline__ void slab_weights(const float4 &v, const float4 &qv, int e, int end,
                                             float mx, float inv_t, double sum,
                                             const uint64_t *tab, float (&w)[4]) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        float x = 0.0f;
        if (e + c < end) {
            const float p = geist_expf_glibc(softmax_arg(f4_get(v, c), mx, inv_t), tab);
            if (RESID) {
                const float r = __fsub_rn((float) ((double) p / sum), f4_get(qv, c));
                x             = r > 0.0f ? r : 0.0f;
            } else {
                x = p;
            }
        }
        w[c] = x;
    }
}

template <int NV>
__device__ __forceinline__ void load_q_chunk(const float *qrow, bool vec, int base, int end,
                                             float4 (&qv)[NV]) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int e = base + 4 * (j * TPB + tid);
        if (vec && e + 3 < end) {
            qv[j] = *reinterpret_cast<const float4 *>(qrow + e);
        } else {
            qv[j].x = e + 0 < end ? qrow[e + 0] : 0.f;
            qv[j].y = e + 1 < end ? qrow[e + 1] : 0.f;
            qv[j].z = e + 2 < end ? qrow[e + 2] : 0.f;
            qv[j].w = e + 3 < end ? qrow[e + 3] : 0.f;
        }
    }
}

/* ---- k_spec_resid ---------------------------------------------------------------------------- */
template <int NV>
__global__ __launch_bounds__(TPB) void k_spec_resid(RowView rv, SpecArgs a) {
    __shared__ SpecShared sh;
    __shared__ double     s_sum[NWAVES];
    __shared__ uint64_t   s_tab[32];
    const int seq = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
    if (tid < 32)
        s_tab[tid] = g_expf_tab[tid];
    const int js = spec_first_reject(rv, a, seq, sh);
    if (a.greedy || js >= a.L)
        return; /* nothing to resample from */
    const long   row = (long) seq * (a.L + 1) + js;
    const float  mx  = key2f(best_key(sh.row_best[js]));
    const double sum = sh.row_sum[js];
    int          base, end;
    chunk_bounds<NV>(rv, chunk, base, end);
    float4       v[NV], qv[NV];
    const float *qrow = a.q + ((long) seq * a.L + js) * a.ld_q;
    const bool   qvec = ((((uintptr_t) a.q) & 15) == 0) && (a.ld_q % 4 == 0);
    load_raw<NV>(rv, rv.logits + row * rv.ld, base, end, v);
    load_q_chunk<NV>(qrow, qvec, base, end, qv);
    double acc = 0.0;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        float w[4];
        slab_weights<true>(v[j], qv[j], base + 4 * (j * TPB + tid), end, mx, a.inv_t, sum, s_tab, w);
        acc += (double) w[0];
        acc += (double) w[1];
        acc += (double) w[2];
        acc += (double) w[3];
    }
    acc = block_sum_f64(acc, s_sum);
    if (tid == 0)
        a.resid_sum[(long) seq * rv.n_chunks + chunk] = acc;
}

/* Index-order walk over one row: locates the chunk from the per-chunk weights, then scans that
 * chunk slab by slab (index order inside a chunk is (slab, thread, component)). Returns the id
 * to every thread; when rounding leaves the target beyond the last weight, the last entry of
 * that chunk with a positive weight (the reference returns the last index, sampler.c:100-101). */
template <int NV, bool RESID>
__device__ int index_order_walk(const RowView &rv, long row, const double *chunk_w, int C,
                                float u, float mx, float inv_t, double sum, const float *qrow,
                                bool qvec, const uint64_t *tab, double *s_scan, int *s_i2,
                                double *s_d2) {
    const int tid = threadIdx.x;
    if (tid == 0) {
        double tot = 0.0;
        for (int c = 0; c < C; ++c)
            tot += chunk_w[c];
        const double target = (double) u * tot;
        double       run    = 0.0;
        int          at     = C - 1;
        for (int c = 0; c < C; ++c) {
            const double nxt = run + chunk_w[c];
            if (target < nxt || c == C - 1) {
                at = c;
                break;
            }
            run = nxt;
        }
        s_i2[0] = at;
        s_i2[1] = 0x7fffffff; /* pick */
        s_i2[2] = -1;         /* last positive */
        s_d2[0] = run;
        s_d2[1] = target;
    }
    __syncthreads();
    const int    chunk  = s_i2[0];
    double       carry  = s_d2[0];
    const double target = s_d2[1];
    int          base, end;
    chunk_bounds<NV>(rv, chunk, base, end);
    float4 v[NV], qv[NV];
    load_raw<NV>(rv, rv.logits + row * rv.ld, base, end, v);
    if (RESID)
        load_q_chunk<NV>(qrow, qvec, base, end, qv);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int e = base + 4 * (j * TPB + tid);
        float     w[4];
        slab_weights<RESID>(v[j], RESID ? qv[j] : v[j], e, end, mx, inv_t, sum, tab, w);
        const double part = (double) w[0] + (double) w[1] + (double) w[2] + (double) w[3];
        double       slab;
        const double incl = block_scan_f64(part, s_scan, &slab);
        double       run  = carry + (incl - part);
        int          lastpos = -1;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            run += (double) w[c];
            if (w[c] > 0.0f)
                lastpos = e + c;
            if (e + c < end && w[c] > 0.0f && target < run) {
                atomicMin(&s_i2[1], e + c);
                break;
            }
        }
        if (lastpos >= 0)
            atomicMax(&s_i2[2], lastpos);
        carry += slab;
    }
    __syncthreads();
    int tok = s_i2[1];
    if (tok == 0x7fffffff)
        tok = s_i2[2] >= 0 ? s_i2[2] : end - 1;
    __syncthreads();
    return tok;
}

/* ---- k_spec_final ---------------------------------------------------------------------------- */
template <int NV>
__global__ __launch_bounds__(TPB) void k_spec_final(RowView rv, SpecArgs a) {
    __shared__ SpecShared sh;
    __shared__ double     s_scan[NWAVES];
    __shared__ double     s_w[MAX_CHUNKS];
    __shared__ uint64_t   s_tab[32];
    __shared__ int        s_i2[4];
    __shared__ double     s_d2[2];
    const int seq = blockIdx.x, tid = threadIdx.x, C = rv.n_chunks, L = a.L;
    if (tid < 32)
        s_tab[tid] = g_expf_tab[tid];
    const int js = spec_first_reject(rv, a, seq, sh);
    if (tid < js)
        a.out_tokens[(long) seq * (L + 1) + tid] = a.draft[(long) seq * L + tid];
    if (tid == 0)
        a.n_accepted[seq] = js;
    const long  row = (long) seq * (L + 1) + js;
    const float u   = a.uniforms[(long) seq * (L + 1) + L];
    int         tok;
    if (a.greedy) {
        const float first = rv.logits[row * rv.ld];
        tok               = (first != first) ? 0 : (int) best_idx(sh.row_best[js]);
    } else {
        const float  mx   = key2f(best_key(sh.row_best[js]));
        const double sum  = sh.row_sum[js];
        bool         resid = js < L;
        if (resid) {
            if (tid < C)
                s_w[tid] = a.resid_sum[(long) seq * C + tid];
            __syncthreads();
            double R = 0.0;
            for (int c = 0; c < C; ++c)
                R += s_w[c];
            resid = R > 0.0; /* p == q everywhere it matters: fall back to a draw from p */
            __syncthreads();
        }
        if (resid) {
            const float *qrow = a.q + ((long) seq * L + js) * a.ld_q;
            const bool   qvec = ((((uintptr_t) a.q) & 15) == 0) && (a.ld_q % 4 == 0);
            tok = index_order_walk<NV, true>(rv, row, s_w, C, u, mx, a.inv_t, sum, qrow, qvec,
                                             s_tab, s_scan, s_i2, s_d2);
        } else {
            if (tid < C)
                s_w[tid] = a.chunk_sum[row * C + tid];
            __syncthreads();
            tok = index_order_walk<NV, false>(rv, row, s_w, C, u, mx, a.inv_t, sum, nullptr, false,
                                              s_tab, s_scan, s_i2, s_d2);
        }
    }
    if (tid == 0)
        a.out_tokens[(long) seq * (L + 1) + js] = tok;
}

} // namespace gs
#endif
