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
 * Kernels (after k_scan_expsum over all n_seq * (L+1) target rows):
 *   k_spec_resid   grid (chunks, n_seq): row sums and maxima, j*, the accepted ids and their
 *                  count (spec_accept_seq), then the sum of max(0, p - q) over its chunk of row j*
 *   k_spec_final   grid (n_seq): draws the last token
 *   k_spec_resid_draw  grid (chunks, n_seq): the two above in one launch, for batches of up to
 *                  two workgroups per compute unit; the chunks of a sequence meet for their
 *                  residual sums and the one in whose chunk the draw falls walks it from registers
 *   k_spec_accept  grid (n_seq): the verdicts alone, for the greedy mode (no residual)
 */
#ifndef GEIST_SAMPLER_SPEC_H
#define GEIST_SAMPLER_SPEC_H

namespace gs {

struct SpecArgs {
    int             L;       /* draft length */
    int             greedy;  /* T <= 0: exact match against the row argmax */
    float           inv_t;
    const float    *q;       /* [n_seq][L][n_vocab], row stride ld_q; NULL = point-mass drafts */
    long            ld_q;
    const int32_t  *draft;   /* [n_seq][L] */
    const float    *uniforms; /* [n_seq][L+1] */
    const uint64_t *chunk_best;
    const double   *chunk_sum;
    const float    *probe_p; /* unnormalised p_j(x_j) per target row */
    double         *resid_sum; /* [n_seq][chunks] */
    double         *resid_slab; /* [n_seq][chunks][SLABS_MAX] */
    const double   *slab_sum;  /* [rows][chunks][SLABS_MAX] of the exp-sum pass, or NULL */
    int32_t        *out_tokens; /* [n_seq][L+1] */
    int32_t        *n_accepted; /* [n_seq] */
};

constexpr int SPEC_L_MAX = 63;

/* The outcome of the acceptance test of one sequence (spec_accept_seq). */
struct SpecVerdict {
    double sum;   /* exp-sum of target row j* */
    float  mx;    /* its maximum */
    int    js;    /* j*: first rejected position, L when every draft token is accepted */
    int    amax;  /* argmax of row j* (greedy mode) */
    int    pad;
};
static_assert(sizeof(SpecVerdict) == SPEC_VERDICT_BYTES, "workspace is sized by the constant");

/* ---- the acceptance test --------------------------------------------------------------------- */
/* By one workgroup, for one sequence. Groups of 16 lanes each take one target row: the lanes share the
 * row's chunks, partial maxima / sums are combined inside the group in a fixed order (DPP row
 * steps). Then lane j of the first wavefront tests position j and a ballot gives j*. */
struct SpecAcceptShared {
    double      sum[SPEC_L_MAX + 1];
    uint64_t    best[SPEC_L_MAX + 1];
    SpecVerdict vd;
};
/* The verdict of sequence `seq`, to every thread of the workgroup. `publish`: this workgroup is
 * the one that writes the accepted ids, their count and the verdict for the kernels behind. */
__device__ __forceinline__ SpecVerdict spec_accept_seq(const RowView &rv, const SpecArgs &a, int seq,
                                                       SpecAcceptShared &sh, bool publish,
                                                       SpecVerdict *verdict) {
    double   *s_sum  = sh.sum;
    uint64_t *s_best = sh.best;
    const int tid = threadIdx.x, C = rv.n_chunks, L = a.L;
    /* what the test of position `tid` needs, asked for before the chunk results: the draft's
     * probability is a read that depends on the draft id, and is under way while those results
     * are fetched and combined */
    int   x  = -1;
    float uu = 0.0f, pp = 0.0f, qt = 0.0f;
    if (tid < L) {
        x = a.draft[(long) seq * L + tid];
        if (!a.greedy) {
            uu = a.uniforms[(long) seq * (L + 1) + tid];
            pp = a.probe_p[(long) seq * (L + 1) + tid];
            if (x >= 0 && x < rv.n_vocab)
                qt = a.q ? a.q[((long) seq * L + tid) * a.ld_q + x] : 1.0f; /* NULL: point mass */
        }
    }
    const int part = tid & 15;
    for (int j = tid >> 4; j <= L; j += TPB / 16) {
        const long row = (long) seq * (L + 1) + j;
        uint64_t   b   = 0;
        double     t   = 0.0;
        for (int c = part; c < C; c += 16) {
            const uint64_t p = a.chunk_best[row * C + c];
            b                = p > b ? p : b;
            if (!a.greedy)
                t += a.chunk_sum[row * C + c];
        }
        /* combine the 16 lanes of the group (one DPP row): lane 15 of the row ends with all */
#define GS_DPP_MAX_U64(ctrl)                                                                    \
    {                                                                                          \
        const uint64_t ob =                                                                    \
            ((uint64_t) (uint32_t) __builtin_amdgcn_update_dpp(0, (int) (b >> 32), ctrl, 0xf, 0xf, \
                                                               false)                          \
             << 32) |                                                                          \
            (uint32_t) __builtin_amdgcn_update_dpp(0, (int) (uint32_t) b, ctrl, 0xf, 0xf, false); \
        b = ob > b ? ob : b;                                                                   \
    }
        GS_DPP_MAX_U64(0x111) /* row_shr:1 */
        GS_DPP_MAX_U64(0x112)
        GS_DPP_MAX_U64(0x114)
        GS_DPP_MAX_U64(0x118)
#undef GS_DPP_MAX_U64
        t += dpp_fetch_f64<0x111, 0xf>(t);
        t += dpp_fetch_f64<0x112, 0xf>(t);
        t += dpp_fetch_f64<0x114, 0xf>(t);
        t += dpp_fetch_f64<0x118, 0xf>(t);
        if (part == 15) {
            s_best[j] = b;
            s_sum[j]  = t;
        }
    }
    __syncthreads();
    if (tid < WAVE) {
    bool ok = true; /* lanes at or beyond L never reject */
    if (tid < L) {
        if (a.greedy) {
            /* a NaN at index 0 keeps the argmax at 0 (sampler.c:52-62) */
            const float first = rv.logits[((long) seq * (L + 1) + tid) * rv.ld];
            ok                = x == ((first != first) ? 0 : (int) best_idx(s_best[tid]));
        } else {
            /* (a draft id outside the vocabulary has q = 0 and p = 0: rejected) */
            const float pn =
                x >= 0 && x < rv.n_vocab ? (float) ((double) pp / s_sum[tid]) : 0.0f;
            ok = (double) uu * (double) qt < (double) pn;
        }
    }
    const uint64_t rej = __ballot(!ok);
    const int      js  = rej ? __ffsll((long long) rej) - 1 : L;
    if (publish && tid < js)
        a.out_tokens[(long) seq * (L + 1) + tid] = x;
    if (tid == 0) {
        /* (the argmax is the greedy mode's answer; only there is the row's first logit read) */
        const float first = a.greedy ? rv.logits[((long) seq * (L + 1) + js) * rv.ld] : 0.0f;
        SpecVerdict v;
        v.sum  = a.greedy ? 0.0 : s_sum[js];
        v.mx   = key2f(best_key(s_best[js]));
        v.js   = js;
        v.amax = (first != first) ? 0 : (int) best_idx(s_best[js]);
        v.pad  = 0;
        sh.vd  = v;
        if (publish) {
            verdict[seq]      = v;
            a.n_accepted[seq] = js;
        }
    }
    }
    __syncthreads();
    return sh.vd;
}

/* the verdicts alone: the greedy mode, which has no residual pass */
__global__ __launch_bounds__(TPB) void k_spec_accept(RowView rv, SpecArgs a, SpecVerdict *verdict) {
    __shared__ SpecAcceptShared sh;
    (void) spec_accept_seq(rv, a, (int) blockIdx.x, sh, true, verdict);
}

/* The residual weights max(0, p - q) of chunk [base, end) of target row `row`, summed per slab
 * over the workgroup: every thread receives the NV slab sums in acc[]; v[] returns the thread's
 * weights themselves (group j: the four elements it owns in slab j), qv[] is scratch. */
template <int NV>
__device__ __forceinline__ void resid_chunk_sums(const RowView &rv, long row, int base, int end,
                                                 const float *qrow, bool qvec, int qx, float mx,
                                                 float inv_t, double sum, const uint64_t *s_tab,
                                                 double *s_sum, float4 (&v)[NV], float4 (&qv)[NV],
                                                 double (&acc)[NV]) {
    const int tid = threadIdx.x;
    load_raw<NV>(rv, rv.logits + row * rv.ld, base, end, v);
    load_q_chunk<NV>(qrow, qvec, qx, base, end, qv);
    apply_transform<NV>(rv, nullptr, v); /* the soft-cap, as in the passes before */
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        float w[4];
        slab_weights<true>(v[j], qv[j], base + 4 * (j * TPB + tid), end, mx, inv_t, sum, s_tab, w);
        acc[j] = (double) w[0];
        acc[j] += (double) w[1];
        acc[j] += (double) w[2];
        acc[j] += (double) w[3];
        v[j] = make_float4(w[0], w[1], w[2], w[3]);
    }
    block_sum_f64_multi<NV>(acc, s_sum);
}

/* ---- k_spec_resid ---------------------------------------------------------------------------- */
template <int NV>
__global__ __launch_bounds__(TPB) void k_spec_resid(RowView rv, SpecArgs a, SpecVerdict *verdict) {
    __shared__ double   s_sum[NWAVES * NV];
    __shared__ uint64_t s_tab[32];
    const int seq = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
    if (tid < 32)
        s_tab[tid] = g_expf_tab[tid];
    /* every workgroup of the sequence works out the verdict for itself (a few hundred chunk
     * results from L2: cheaper than a kernel of its own in front of this one); the first one
     * leaves it for k_spec_final */
    __shared__ SpecAcceptShared s_acc;
    const SpecVerdict vd = spec_accept_seq(rv, a, seq, s_acc, chunk == 0, verdict);
    const int         js = vd.js;
    if (a.greedy || js >= a.L)
        return; /* nothing to resample from */
    const long   row = (long) seq * (a.L + 1) + js;
    const float  mx  = vd.mx;
    const double sum = vd.sum;
    int base, end;
    chunk_bounds<NV>(rv, chunk, base, end);
    float4       v[NV], qv[NV];
    const float *qrow = a.q ? a.q + ((long) seq * a.L + js) * a.ld_q : nullptr;
    const bool   qvec = ((((uintptr_t) a.q) & 15) == 0) && (a.ld_q % 4 == 0);
    const int    qx   = a.draft[(long) seq * a.L + js];
    double       acc[NV];
    resid_chunk_sums<NV>(rv, row, base, end, qrow, qvec, qx, mx, a.inv_t, sum, s_tab, s_sum, v, qv,
                         acc);
    if (tid == 0) {
        const long at  = (long) seq * rv.n_chunks + chunk;
        double     tot = 0.0;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            a.resid_slab[at * SLABS_MAX + j] = acc[j];
            tot += acc[j];
        }
        a.resid_sum[at] = tot;
    }
}

/* A draw from p of target row `row` (the bonus token, or the fallback when the residual is
 * empty): the temperature walk over the sums the exp-sum pass left. `s_w`: MAX_CHUNKS doubles. */
template <int NV>
__device__ __forceinline__ int spec_draw_from_p(const RowView &rv, const SpecArgs &a, long row,
                                                float u, float mx, double sum, double *s_w,
                                                const uint64_t *s_tab, WalkShared &s_walk) {
    const int tid = threadIdx.x, C = rv.n_chunks;
    if (tid < C)
        s_w[tid] = a.chunk_sum[row * C + tid];
    __syncthreads();
    /* (the exp-sum pass of the verification keeps no slab sums: few rows are drawn from, and
     * those by a workgroup that has nothing else to do) */
    return index_order_walk<NV, false, false>(
        rv, (int) row, 0, s_w, a.slab_sum ? a.slab_sum + row * C * SLABS_MAX : nullptr, C, u, mx,
        a.inv_t, sum, nullptr, false, -1, s_tab, nullptr, s_walk);
}

/* ---- k_spec_final ---------------------------------------------------------------------------- */
template <int NV>
__global__ __launch_bounds__(TPB) void k_spec_final(RowView rv, SpecArgs a,
                                                    const SpecVerdict *__restrict__ verdict) {
    __shared__ WalkShared s_walk;
    __shared__ double     s_w[MAX_CHUNKS];
    __shared__ uint64_t   s_tab[32];
    const int seq = blockIdx.x, tid = threadIdx.x, C = rv.n_chunks, L = a.L;
    if (tid < 32)
        s_tab[tid] = g_expf_tab[tid];
    const SpecVerdict vd  = verdict[seq];
    const int         js  = vd.js;
    const long        row = (long) seq * (L + 1) + js;
    const float       u   = a.uniforms[(long) seq * (L + 1) + L];
    int               tok;
    if (a.greedy) {
        tok = vd.amax;
    } else {
        const float  mx    = vd.mx;
        const double sum   = vd.sum;
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
            const float *qrow = a.q ? a.q + ((long) seq * L + js) * a.ld_q : nullptr;
            const bool   qvec = ((((uintptr_t) a.q) & 15) == 0) && (a.ld_q % 4 == 0);
            const int    qx   = a.draft[(long) seq * L + js];
            tok = index_order_walk<NV, false, true>(rv, (int) row, 0, s_w,
                                                    a.resid_slab + (long) seq * C * SLABS_MAX, C, u,
                                                    mx, a.inv_t, sum, qrow, qvec, qx, s_tab,
                                                    nullptr, s_walk);
        } else {
            tok = spec_draw_from_p<NV>(rv, a, row, u, mx, sum, s_w, s_tab, s_walk);
        }
    }
    if (tid == 0)
        a.out_tokens[(long) seq * (L + 1) + js] = tok;
}

/* ---- k_spec_resid_draw ----------------------------------------------------------------------- */
/* k_spec_resid and k_spec_final in one launch (stochastic verification only). The workgroups of
 * a sequence work out the verdict, sum the residual of their chunks, and meet for those sums
 * (row_sums_meet, as the temperature draw's workgroups do); each then adds them up in chunk
 * order and locates the draw with the same arithmetic on the same numbers, so exactly one finds
 * it in its own chunk and walks that chunk from the registers it still holds. The sums, the
 * location and the walk are those of the two kernels (resid_chunk_sums, walk_locate_chunk,
 * walk_slab_step), so the token is the same bit for bit. A sequence whose drafts are all accepted,
 * or whose residual is empty, has its token drawn from p by its first workgroup, from the sums of
 * the exp-sum pass. A workgroup that gives up the wait forms the other chunks' sums itself (the
 * same summation, so it still agrees with the others on the chunk) and walks from memory. */
template <int NV>
__global__ __launch_bounds__(TPB) void k_spec_resid_draw(RowView rv, SpecArgs a,
                                                         SpecVerdict *verdict, MeetSpace meet) {
    __shared__ double           s_sum[NWAVES * NV];
    __shared__ uint64_t         s_tab[32];
    __shared__ SpecAcceptShared s_acc;
    __shared__ DrawShared       s_draw;
    const int seq = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x, C = rv.n_chunks, L = a.L;
    if (tid < 32)
        s_tab[tid] = g_expf_tab[tid];
    {
        const uint32_t wg = blockIdx.y * gridDim.x + blockIdx.x, n_wg = gridDim.x * gridDim.y;
        for (uint32_t i = wg * TPB + tid; i < meet.stale_count; i += n_wg * TPB)
            meet.stale[i] = 0;
    }
    const SpecVerdict vd  = spec_accept_seq(rv, a, seq, s_acc, chunk == 0, verdict);
    const int         js  = vd.js;
    const long        row = (long) seq * (L + 1) + js;
    const float       u   = a.uniforms[(long) seq * (L + 1) + L];
    const float       mx  = vd.mx;
    const double      sum = vd.sum;
    if (js >= L) { /* every draft accepted: the bonus token, a draw from p_L */
        if (chunk != 0)
            return;
        const int tok = spec_draw_from_p<NV>(rv, a, row, u, mx, sum, s_draw.csum, s_tab, s_draw.walk);
        if (tid == 0)
            a.out_tokens[row] = tok;
        return;
    }
    int base, end;
    chunk_bounds<NV>(rv, chunk, base, end);
    float4       v[NV], qv[NV];
    const float *qrow = a.q ? a.q + ((long) seq * L + js) * a.ld_q : nullptr;
    const bool   qvec = ((((uintptr_t) a.q) & 15) == 0) && (a.ld_q % 4 == 0);
    const int    qx   = a.draft[(long) seq * L + js];
    double       acc[NV];
    resid_chunk_sums<NV>(rv, row, base, end, qrow, qvec, qx, mx, a.inv_t, sum, s_tab, s_sum, v, qv,
                         acc);
    if (tid == 0) {
        double tot = 0.0;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            s_draw.slab[j] = acc[j];
            tot += acc[j];
        }
        s_draw.total = tot;
    }
    __syncthreads();
    row_sums_meet(meet.slots + (long) seq * C, chunk, C, s_draw.total, tid < WAVE, true,
                  meet.wait_limit, s_draw);
    const bool from_registers = s_draw.have_sums != 0;
    if (!from_registers) {
        /* not met: every other chunk's sum by this workgroup, with the same summation */
        if (tid == 0)
            s_draw.csum[chunk] = s_draw.total;
        for (int c2 = 0; c2 < C; ++c2) {
            if (c2 == chunk)
                continue;
            int b2, e2;
            chunk_bounds<NV>(rv, c2, b2, e2);
            double acc2[NV];
            resid_chunk_sums<NV>(rv, row, b2, e2, qrow, qvec, qx, mx, a.inv_t, sum, s_tab, s_sum, v,
                                 qv, acc2);
            if (tid == 0) {
                double tot = 0.0;
#pragma unroll
                for (int j = 0; j < NV; ++j)
                    tot += acc2[j];
                s_draw.csum[c2] = tot;
            }
        }
        __syncthreads();
    }
    /* the residual's mass, added up as k_spec_final adds it */
    double R = 0.0;
    for (int c = 0; c < C; ++c)
        R += s_draw.csum[c];
    if (!(R > 0.0)) { /* p == q everywhere it matters: a draw from p */
        if (chunk != 0)
            return;
        __syncthreads(); /* csum is about to hold the sums of p */
        const int tok = spec_draw_from_p<NV>(rv, a, row, u, mx, sum, s_draw.csum, s_tab, s_draw.walk);
        if (tid == 0)
            a.out_tokens[row] = tok;
        return;
    }
    /* where the draw falls: the same arithmetic in every workgroup of the sequence */
    if (tid < WAVE) {
        double    run, target;
        const int at = walk_locate_chunk(s_draw.csum, C, u, &run, &target);
        int       sl = 0;
        if (at == chunk)
            sl = walk_locate_slab<NV>(s_draw.slab, target, &run);
        if (tid == 0) {
            s_draw.walk.chunk    = at;
            s_draw.walk.slab     = sl;
            s_draw.walk.before   = run;
            s_draw.walk.target   = target;
            s_draw.walk.pick     = 0x7fffffff;
            s_draw.walk.last_pos = -1;
        }
    }
    __syncthreads();
    if (s_draw.walk.chunk != chunk)
        return; /* another workgroup's */
    const double target = s_draw.walk.target;
    double       carry  = s_draw.walk.before;
    const int    sl     = __builtin_amdgcn_readfirstlane(s_draw.walk.slab);
    int          end_w  = end;
    bool         found  = false;
    if (from_registers) {
        /* the located slab's weights, which the summation left in the registers: nothing is
         * computed again. Should rounding have left the target beyond the slab, the walk goes
         * on through the row from memory. */
        float4 vs = v[0];
#pragma unroll
        for (int j = 1; j < NV; ++j)
            if (j == sl)
                vs = v[j];
        const int   sbase = base + sl * 4 * TPB;
        const int   send  = sbase + 4 * TPB < end ? sbase + 4 * TPB : end;
        const int   e     = sbase + 4 * tid;
        const float w[4]  = {vs.x, vs.y, vs.z, vs.w};
        found = walk_slab_step<true>(w, e, send, target, carry, s_draw.walk);
        if (!found)
            walk_from<NV, false, true>(rv, (int) row, 0, C, chunk, sl + 1, carry, target, mx,
                                       a.inv_t, sum, qrow, qvec, qx, s_tab, nullptr, s_draw.walk,
                                       end_w);
    } else {
        walk_from<NV, false, true>(rv, (int) row, 0, C, chunk, sl, carry, target, mx, a.inv_t, sum,
                                   qrow, qvec, qx, s_tab, nullptr, s_draw.walk, end_w);
    }
    __syncthreads();
    int tok = s_draw.walk.pick;
    if (tok == 0x7fffffff)
        tok = s_draw.walk.last_pos >= 0 ? s_draw.walk.last_pos : end_w - 1;
    if (tid == 0)
        a.out_tokens[row] = tok;
}

} // namespace gs
#endif
