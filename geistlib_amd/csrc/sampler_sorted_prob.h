/*
 * sampler_sorted_prob.h -- the full-vocabulary probability-ordered modes: top-p (the
 * reference's geist_sampler_top_p_ws, src/engine/sampler.c:232-305) and min-p, without a
 * top-k in front. Included by sampler_kernels.hip.
 *
 * The reference normalises every probability, sorts all of them and walks the sorted list.
 * Here nothing is sorted but the few entries that can matter; a row takes the cheapest of three
 * walks that can certify its result, decided on the device through the row's flag:
 *   shortcut (k_final_sorted)    thread maxima -> a logit bound below which nothing of the kept
 *                                prefix can lie -> re-read the threads above it -> order those
 *                                entries -> walk. Kept prefixes of up to about a hundred.
 *   list (flag 1 or 4: k_list_candidates / the exp-sum pass, k_sorted_candidates)
 *                                every element up to a z bin is listed with its normalised
 *                                probability; one mass histogram over the list locates the
 *                                nucleus edge and the draw. Kept prefixes of thousands.
 *   whole row (flag 2: sorted_general_row)  the row's probabilities are written once, then a
 *                                mass-weighted radix descent over their bit patterns finds the
 *                                edge and the drawn entry. Anything else.
 */
#ifndef GEIST_SAMPLER_SORTED_PROB_H
#define GEIST_SAMPLER_SORTED_PROB_H

namespace gs {

/* Walk over n <= 64 * IPT entries already in walk order, on ONE wavefront: entry i carries
 * its weight pn_i as the high word of spack[i] (fp32 bits; positive floats order like their
 * bits) and its vocabulary id in the low word (complemented, as pack_best()).
 * Nucleus: sampler.c:273-283; min-p: pn >= min_p * pn_0; draw: sampler.c:286-299.
 * Returns the vocabulary id, or -1 when top_p is set, min_p is not, and the n entries do not
 * reach top_p (the caller's bound was too tight). */
template <int IPT>
__device__ int finish_weights_wave(int n, const uint64_t *spack, float top_p, float min_p,
                                   float u) {
    const int  lane  = threadIdx.x & (WAVE - 1);
    const bool use_p = top_p > 0.0f && top_p < 1.0f;
    const bool use_m = min_p > 0.0f;
    float      w[IPT];
    double     part = 0.0;
#pragma unroll
    for (int t = 0; t < IPT; ++t) {
        const int i = IPT * lane + t;
        w[t]        = i < n ? __uint_as_float(best_key(spack[i])) : 0.0f;
        part += (double) w[t];
    }
    const double incl = wave_scan_f64_dpp(part);
    double       c[IPT];
    {
        double run = incl - part;
#pragma unroll
        for (int t = 0; t < IPT; ++t) {
            run += (double) w[t];
            c[t] = run;
        }
    }
    int keep = n;
    if (use_p) {
        int first = 0x7fffffff;
#pragma unroll
        for (int t = IPT - 1; t >= 0; --t) {
            const uint64_t mk = __ballot(IPT * lane + t < n && c[t] >= (double) top_p);
            if (mk) {
                const int f = IPT * (__ffsll((long long) mk) - 1) + t;
                first       = f < first ? f : first;
            }
        }
        if (first != 0x7fffffff)
            keep = first + 1;
        else if (!use_m)
            return -1;
    }
    if (use_m) {
        const float floor_w = __fmul_rn(min_p, __shfl(w[0], 0, WAVE));
        int         m       = 0;
#pragma unroll
        for (int t = 0; t < IPT; ++t)
            m += __popcll(__ballot(IPT * lane + t < n && w[t] >= floor_w));
        if (m < 1)
            m = 1;
        keep = m < keep ? m : keep;
    }
    if (keep < 1)
        keep = 1;
    double at_keep = c[0];
#pragma unroll
    for (int t = 1; t < IPT; ++t)
        if (((keep - 1) % IPT) == t)
            at_keep = c[t];
    const double mass   = __shfl(at_keep, (keep - 1) / IPT, WAVE);
    const double target = (double) u * mass;
    int          at     = 0x7fffffff;
#pragma unroll
    for (int t = IPT - 1; t >= 0; --t) {
        const uint64_t hk = __ballot(IPT * lane + t < keep && target < c[t]);
        if (hk) {
            const int f = IPT * (__ffsll((long long) hk) - 1) + t;
            at          = f < at ? f : at;
        }
    }
    if (at == 0x7fffffff)
        at = keep - 1;
    return (int) best_idx(spack[at]);
}

/* ============================================================================================
 * sorted_from_tmax: fast path. `mx` is the row maximum, `sum` the row's double sum of
 * expf((l - mx) * inv_t) (both from the streaming kernels). Steps:
 *   1. thread maxima -> each thread of this workgroup keeps the largest of its KPT and its
 *      normalised probability w;
 *   2. top-p: the elements at or above a logit t weigh at least the sum of w over the threads
 *      whose maximum is >= t (one distinct element each), so the largest t for which that sum
 *      reaches top_p bounds the nucleus from below; found by a bitwise search on the key.
 *      min-p: pn_i >= min_p * pn_0 needs (l_i - mx) * inv_t >= ln(min_p), a bound in closed
 *      form (taken with slack). Both set: the kept prefix is the shorter one, so the larger
 *      bound serves;
 *   3. re-read the threads at or above the bound, transform, keep the entries above it with
 *      their exact pn = (float)((double)p / sum) (sampler.c:251-253);
 *   4. order by (pn descending, index ascending) (sampler.c:270) and walk.
 * Returns the vocabulary id, or -1 when the row has to take the general path.
 * ========================================================================================== */
template <int NV, bool PEN, int KPT>
__device__ __forceinline__ int sorted_from_tmax(const RowView &rv, const FinalArgs &a, int row,
                                                float mx, double sum, float u_row, uint8_t *slot,
                                                uint32_t *s_mx, float *s_wt, int *s_selid,
                                                uint32_t *s_pcnt, uint64_t *s_m, uint64_t *s_srt,
                                                int *s_n, int *s_n2, const uint64_t *tab) {
    const int  tid = threadIdx.x, lane = tid & (WAVE - 1);
    const int  C     = rv.n_chunks;
    const bool use_p = a.top_p > 0.0f && a.top_p < 1.0f;
    const bool use_m = a.min_p > 0.0f;
    HistPrefetch pf;
    if (PEN)
        pf = history_prefetch(rv, row, rv.n_rows);
    /* 1 */
    const float *tm = a.tmax + (long) row * C * TPB + tid;
    float        raw[KPT];
#pragma unroll
    for (int q = 0; q < KPT; ++q)
        raw[q] = q < C ? tm[q * TPB] : __builtin_nanf("");
    {
        uint4 *z = reinterpret_cast<uint4 *>(slot);
        for (int i = tid; i < KPT * TPB / 16; i += TPB)
            z[i] = make_uint4(0u, 0u, 0u, 0u);
        if (PEN) {
            uint4 *zc = reinterpret_cast<uint4 *>(s_pcnt);
            for (int i = tid; i < SEL_MAX * NV; i += TPB)
                zc[i] = make_uint4(0u, 0u, 0u, 0u);
        }
        if (tid == 0) {
            *s_n  = 0;
            *s_n2 = 0;
        }
    }
    float mxf = __builtin_nanf("");
#pragma unroll
    for (int q = 0; q + 1 < KPT; q += 2)
        mxf = max3f(mxf, raw[q], raw[q + 1]);
    const uint32_t mkey = f2key(mxf);
    float          wt   = 0.0f;
    if (mkey)
        wt = (float) ((double) geist_expf_glibc_le0(softmax_arg(mxf, mx, a.inv_t), tab) / sum);
    s_mx[tid] = mkey;
    s_wt[tid] = wt;
    __syncthreads();
    /* 2 */
    uint32_t key_lo = 0u;
    if (use_p) {
        const uint32_t k0 = s_mx[lane], k1 = s_mx[lane + 64], k2 = s_mx[lane + 128],
                       k3 = s_mx[lane + 192];
        const float w0 = s_wt[lane], w1 = s_wt[lane + 64], w2 = s_wt[lane + 128],
                    w3 = s_wt[lane + 192];
        /* fp32 sums of at most 256 terms: ask for a little more than top_p */
        const float need = a.top_p * 1.0001f;
        uint32_t    tau  = 0u;
#pragma unroll 1
        for (int bit = 31; bit >= 14; --bit) {
            const uint32_t t = tau | (1u << bit);
            float acc = (k0 >= t ? w0 : 0.f) + (k1 >= t ? w1 : 0.f) + (k2 >= t ? w2 : 0.f) +
                        (k3 >= t ? w3 : 0.f);
            acc = wave_sum_f32_dpp(acc);
            if (acc >= need)
                tau = t;
        }
        if (tau < 0x00800000u && !use_m)
            return -1; /* the thread maxima alone do not weigh top_p: a wide nucleus */
        key_lo = tau;
    }
    if (use_m) {
        /* (l - mx) * inv_t >= ln(min_p) - slack  <=>  l >= mx + (ln(min_p) - slack) / inv_t */
        const double   lg  = a.ln_min_p - 1e-3;
        const float    t_m = (float) ((double) mx + lg / (double) a.inv_t - 1e-3 * fabs((double) mx));
        const uint32_t km  = f2key(t_m);
        key_lo             = km > key_lo ? km : key_lo;
    }
    if (key_lo < 0x00800000u)
        return -1;
    const float bound = key2f(key_lo);
    /* 3 */
    uint32_t selmask = 0u;
#pragma unroll
    for (int q = 0; q < KPT; ++q)
        selmask |= (uint32_t) (raw[q] >= bound) << q;
    int pos = wave_reserve(__popc(selmask), s_n);
    while (selmask) {
        const int q = __ffs(selmask) - 1;
        selmask &= selmask - 1u;
        if (pos < SEL_MAX) {
            s_selid[pos]        = q * TPB + tid;
            slot[q * TPB + tid] = (uint8_t) (pos + 1);
        }
        ++pos;
    }
    __syncthreads();
    const int n_sel = *s_n;
    if (n_sel > SEL_MAX)
        return -1;
    constexpr int TASKS = SEL_MAX * NV / TPB;
    float4        r[TASKS];
    int           e0[TASKS], e1[TASKS];
    const float  *rowp = rv.logits + (long) row * rv.ld;
#pragma unroll
    for (int q = 0; q < TASKS; ++q) {
        const int t = tid + q * TPB;
        const int s = t / NV, j = t % NV;
        e0[q] = 0;
        e1[q] = 0;
        r[q]  = make_float4(0.f, 0.f, 0.f, 0.f);
        if (s < n_sel) {
            const int L = s_selid[s];
            const int chunk = L / TPB, tt = L % TPB;
            int       base, end;
            chunk_bounds<NV>(rv, chunk, base, end);
            const int e = base + 4 * (j * TPB + tt);
            e0[q] = e;
            e1[q] = end;
            if (rv.vec_ok && e + 3 < end) {
                r[q] = *reinterpret_cast<const float4 *>(rowp + e);
            } else {
                r[q].x = e + 0 < end ? rowp[e + 0] : 0.f;
                r[q].y = e + 1 < end ? rowp[e + 1] : 0.f;
                r[q].z = e + 2 < end ? rowp[e + 2] : 0.f;
                r[q].w = e + 3 < end ? rowp[e + 3] : 0.f;
            }
        }
    }
    if (PEN) {
        const int shift = 31 - __clz(rv.per_chunk);
        history_for_each_batched(
            rv, row, pf,
            [&](int t) -> int { /* 1 + index of the element's counter, 0 = not gathered */
                if (t < 0 || t >= rv.n_vocab)
                    return 0;
                const int off = t & (rv.per_chunk - 1);
                const int f   = off >> 2;
                const int s   = slot[(t >> shift) * TPB + (f % TPB)];
                return s ? 1 + ((s - 1) * NV + f / TPB) * 4 + (off & 3) : 0;
            },
            [&](int code) {
                if (code)
                    atomicAdd(&s_pcnt[code - 1], 1u);
            });
        __syncthreads();
    }
    /* survivors are appended in any order: the ranking below orders them */
#pragma unroll
    for (int q = 0; q < TASKS; ++q) {
        const int t = tid + q * TPB;
        if (e0[q] >= e1[q])
            continue;
        uint4 hc = make_uint4(0u, 0u, 0u, 0u);
        if (PEN)
            hc = *reinterpret_cast<const uint4 *>(&s_pcnt[t * 4]);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            if (e0[q] + c < e1[q]) {
                float x = f4_get(r[q], c);
                if (PEN) {
                    const uint32_t n_hist = c == 0 ? hc.x : c == 1 ? hc.y : c == 2 ? hc.z : hc.w;
                    if (n_hist)
                        x = penalise(x, n_hist, rv.rep, rv.inv_rep, rv.freq, rv.pres);
                }
                if (rv.softcap > 0.0f)
                    x = softcap1(x, rv.softcap);
                if (rv.allowed && !allowed_at(rv, row, e0[q] + c))
                    continue;
                if (x >= bound) { /* the logit for now; its probability below, one per thread */
                    const int at = atomicAdd(s_n2, 1);
                    if (at < TPB)
                        s_m[at] = ((uint64_t) __float_as_uint(x) << 32) | (uint32_t) (e0[q] + c);
                }
            }
        }
    }
    __syncthreads();
    const int m = *s_n2;
    if (m > TPB || m < 1)
        return -1;
    if (tid < m) {
        const uint64_t ent = s_m[tid];
        const float    x   = __uint_as_float((uint32_t) (ent >> 32));
        const float    pn  =
            (float) ((double) geist_expf_glibc_le0(softmax_arg(x, mx, a.inv_t), tab) / sum);
        s_m[tid] = pack_best(__float_as_uint(pn), (uint32_t) ent);
    }
    __syncthreads();
    /* 4: order by counting, entry i compared by P = 256 / m2 <= 64 neighbouring lanes */
    int m2 = 4;
    while (m2 < m)
        m2 <<= 1;
    const int P = TPB / m2, i = tid / P, part = tid % P;
    uint64_t  me   = 0;
    int       rank = 0;
    if (i < m) {
        me = s_m[i];
#pragma unroll 4
        for (int j = part; j < m; j += P)
            rank += s_m[j] > me;
    }
    for (int d = 1; d < P; d <<= 1)
        rank += __shfl_xor(rank, d, WAVE);
    if (i < m && part == 0)
        s_srt[rank] = me;
    __syncthreads();
    int tok = 0;
    if (tid < WAVE) {
        if (m <= WAVE)
            tok = finish_weights_wave<1>(m, s_srt, a.top_p, a.min_p, u_row);
        else if (m <= 2 * WAVE)
            tok = finish_weights_wave<2>(m, s_srt, a.top_p, a.min_p, u_row);
        else
            tok = finish_weights_wave<4>(m, s_srt, a.top_p, a.min_p, u_row);
    }
    if (tid == 0)
        *s_n = tok;
    __syncthreads();
    tok = *s_n;
    __syncthreads();
    return tok;
}

/* ============================================================================================
 * The whole-row walk: rows the fast path handed on (row_flag != 0). One workgroup per row works
 * on the row's normalised probabilities pn (written by k_write_probs).
 *
 * The sorted order of the reference (pn descending, equal pn by ascending index) is never
 * materialised. A descent over the bit pattern of pn -- 11, 11 and 10 bits per level, each
 * level one pass building a histogram of entry counts and of mass per digit -- finds the value
 * kappa at which the running mass of the sorted list first reaches a target, the mass and count
 * strictly above kappa, and how many of the entries equal to kappa are needed. Mass is summed
 * in 2^-62 fixed point, so the result does not depend on the order of the atomic additions.
 * Two descents: the nucleus edge (target top_p), then the draw (target u * kept mass). A last
 * pass in index order finds the j-th entry equal to the drawn value.
 * ========================================================================================== */
constexpr int SG_BINS = 2048;

struct SortedGenShared {
    uint32_t cnt[SG_BINS];
    uint64_t mass[SG_BINS];
    uint64_t scan64[NWAVES];
    uint32_t scan32[NWAVES];
    uint64_t res_mass_above;
    uint32_t res_cnt_above;
    int      res_digit;
    uint64_t red64[NWAVES];
};

__device__ __forceinline__ uint64_t pn_fx(float pn) {
    return (uint64_t) __double2ull_rz((double) pn * 0x1p62);
}

__device__ __forceinline__ uint64_t block_sum_u64(uint64_t v, uint64_t *scratch) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1)
        v += shfl_xor_u64(v, m);
    if ((threadIdx.x & (WAVE - 1)) == 0)
        scratch[threadIdx.x / WAVE] = v;
    __syncthreads();
    uint64_t r = 0;
#pragma unroll
    for (int w = 0; w < NWAVES; ++w)
        r += scratch[w];
    __syncthreads();
    return r;
}

/* f(i, pn[i]) for every i < n, the workgroup's threads sharing the entries. Many loads of a
 * thread are in flight together (eight of 16 bytes where pn is aligned, eight words otherwise):
 * with one load and its use per turn a pass over a row of 128 k probabilities is 500 round
 * trips to L2 one after the other, and the whole-row walk makes seven such passes; this way a
 * pass that adds nothing to a histogram takes 16 us, about what one compute unit reads from L2.
 * (The order in which entries are visited does not matter to the callers: integer sums and
 * maxima.) */
template <typename F>
__device__ __forceinline__ void for_each_entry(const float *pn, int n, F &&f) {
    int i = 0;
    if ((((uintptr_t) pn) & 15) == 0) {
        const float4 *p4 = reinterpret_cast<const float4 *>(pn);
        const int     n4 = n >> 2;
        int           g  = threadIdx.x;
        for (; g + 7 * TPB < n4; g += 8 * TPB) {
            float4 p[8];
#pragma unroll
            for (int k = 0; k < 8; ++k)
                p[k] = p4[g + k * TPB];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int e = 4 * (g + k * TPB);
                f(e, p[k].x);
                f(e + 1, p[k].y);
                f(e + 2, p[k].z);
                f(e + 3, p[k].w);
            }
        }
        for (; g < n4; g += TPB) {
            const float4 q = p4[g];
            f(4 * g, q.x);
            f(4 * g + 1, q.y);
            f(4 * g + 2, q.z);
            f(4 * g + 3, q.w);
        }
        i = n4 << 2;
    }
    i += threadIdx.x;
    for (; i + 7 * TPB < n; i += 8 * TPB) {
        float p[8];
#pragma unroll
        for (int k = 0; k < 8; ++k)
            p[k] = pn[i + k * TPB];
#pragma unroll
        for (int k = 0; k < 8; ++k)
            f(i + k * TPB, p[k]);
    }
    for (; i < n; i += TPB)
        f(i, pn[i]);
}

/* The digit of a level's histogram (sh.cnt / sh.mass, complete and published by a barrier) at
 * which the running mass, counted from the largest digit down and starting from mass_above,
 * first reaches `target`: sh.res_digit (-1: not reached), sh.res_mass_above and
 * sh.res_cnt_above (strictly greater digits, on top of mass_above / cnt_above). Called by every
 * thread of the workgroup; ends with a barrier. */
__device__ __forceinline__ void sg_select_digit(SortedGenShared &sh, uint64_t target,
                                                uint64_t mass_above, uint32_t cnt_above) {
    const int tid = threadIdx.x;
    /* thread t owns the 8 digits SG_BINS-1-8t .. SG_BINS-8-8t, i.e. descending order */
    uint64_t lm = 0;
    uint32_t lc = 0;
#pragma unroll
    for (int q = 0; q < SG_BINS / TPB; ++q) {
        const int d = SG_BINS - 1 - (tid * (SG_BINS / TPB) + q);
        lm += sh.mass[d];
        lc += sh.cnt[d];
    }
    /* exclusive prefix over threads (descending digits) */
    uint64_t im = lm;
    uint32_t ic = lc;
    {
        const int lane = tid & (WAVE - 1), w = tid / WAVE;
#pragma unroll
        for (int d = 1; d < WAVE; d <<= 1) {
            const uint64_t om = ((uint64_t) (uint32_t) __shfl_up((int) (im >> 32), d, WAVE) << 32) |
                                (uint32_t) __shfl_up((int) (uint32_t) im, d, WAVE);
            const uint32_t oc = (uint32_t) __shfl_up((int) ic, d, WAVE);
            if (lane >= d) {
                im += om;
                ic += oc;
            }
        }
        if (lane == WAVE - 1) {
            sh.scan64[w] = im;
            sh.scan32[w] = ic;
        }
        if (tid == 0)
            sh.res_digit = -1;
        __syncthreads();
        for (int x = 0; x < w; ++x) {
            im += sh.scan64[x];
            ic += sh.scan32[x];
        }
    }
    uint64_t run_m = mass_above + (im - lm);
    uint32_t run_c = cnt_above + (ic - lc);
#pragma unroll
    for (int q = 0; q < SG_BINS / TPB; ++q) {
        const int      d  = SG_BINS - 1 - (tid * (SG_BINS / TPB) + q);
        const uint64_t bm = sh.mass[d];
        if (sh.cnt[d] && run_m < target && run_m + bm >= target) {
            sh.res_digit      = d;
            sh.res_mass_above = run_m;
            sh.res_cnt_above  = run_c;
        }
        run_m += bm;
        run_c += sh.cnt[d];
    }
    __syncthreads();
}

/* One descent. `limit_key`/`limit_ties`: only entries that precede the (limit_key, limit_ties)
 * edge of a previous descent take part -- entries with key > limit_key, plus the first
 * limit_ties (by index) of those equal to it, whose mass is limit_ties * fx(limit_key); pass
 * limit_key = 0, limit_ties = 0 with `limited` false for no restriction.
 * Out: kappa (key bits), cnt_above / mass_above (strictly greater keys), ties_total.
 * Returns false when the whole (restricted) list weighs less than the target. */
__device__ bool sg_descent(const float *pn, int n, uint64_t target, bool limited,
                           uint32_t limit_key, uint32_t limit_ties, SortedGenShared &sh,
                           uint32_t &kappa, uint32_t &cnt_above, uint64_t &mass_above,
                           uint32_t &ties_total) {
    const int tid    = threadIdx.x;
    uint32_t  prefix = 0u, mask = 0u;
    cnt_above  = 0u;
    mass_above = 0ull;
    ties_total = 0u;
    const int shifts[3] = {21, 10, 0};
    const int widths[3] = {11, 11, 10};
    for (int lv = 0; lv < 3; ++lv) {
        const int      shf = shifts[lv];
        const uint32_t dm  = (1u << widths[lv]) - 1u;
        for (int i = tid; i < SG_BINS; i += TPB) {
            sh.cnt[i]  = 0u;
            sh.mass[i] = 0ull;
        }
        __syncthreads();
        for_each_entry(pn, n, [&](int, float p) {
            const uint32_t key = __float_as_uint(p);
            if ((key & mask) != prefix)
                return;
            if (limited && key <= limit_key)
                return; /* entries equal to the limit are added below, as a block */
            const uint32_t d = (key >> shf) & dm;
            atomicAdd(&sh.cnt[d], 1u);
            atomicAdd((unsigned long long *) &sh.mass[d], (unsigned long long) pn_fx(p));
        });
        if (limited && tid == 0 && limit_ties && (limit_key & mask) == prefix) {
            const uint32_t d = (limit_key >> shf) & dm;
            atomicAdd(&sh.cnt[d], limit_ties);
            atomicAdd((unsigned long long *) &sh.mass[d],
                      (unsigned long long) (pn_fx(__uint_as_float(limit_key)) * limit_ties));
        }
        __syncthreads();
        sg_select_digit(sh, target, mass_above, cnt_above);
        const int d = sh.res_digit;
        if (d < 0)
            return false;
        mass_above = sh.res_mass_above;
        cnt_above  = sh.res_cnt_above;
        ties_total = sh.cnt[d];
        prefix |= (uint32_t) d << shf;
        mask |= dm << shf;
        __syncthreads();
    }
    kappa = prefix;
    return true;
}

/* The j-th smallest id among the list entries whose key equals `key`, ids < 2^21: two counting
 * passes over the bits of the id (the list is in no particular order). */
__device__ int list_jth_id(const float *pn, const uint32_t *ids, int n, uint32_t key, int j,
                           SortedGenShared &sh, int *s_scan, int *s_pick) {
    const int tid    = threadIdx.x;
    uint32_t  prefix = 0u;
    int       want   = j; /* 1-based rank inside the current digit range */
    for (int lv = 0; lv < 2; ++lv) {
        for (int i = tid; i < SG_BINS; i += TPB)
            sh.cnt[i] = 0u;
        if (tid == 0)
            *s_pick = -1;
        __syncthreads();
        for (int i = tid; i < n; i += TPB) {
            if (__float_as_uint(pn[i]) != key)
                continue;
            const uint32_t id = ids[i];
            if (lv == 1 && (id >> 10) != prefix)
                continue;
            atomicAdd(&sh.cnt[lv == 0 ? (id >> 10) & (SG_BINS - 1) : id & 1023u], 1u);
        }
        __syncthreads();
        constexpr int PER = SG_BINS / TPB; /* ascending digits */
        int           mine = 0;
#pragma unroll
        for (int q = 0; q < PER; ++q)
            mine += (int) sh.cnt[tid * PER + q];
        const int incl = block_scan_i32(mine, s_scan, nullptr);
        int       run  = incl - mine;
        if (run < want && incl >= want) {
#pragma unroll
            for (int q = 0; q < PER; ++q) {
                const int c = (int) sh.cnt[tid * PER + q];
                if (run < want && run + c >= want) {
                    *s_pick       = tid * PER + q;
                    sh.res_digit  = run;
                }
                run += c;
            }
        }
        __syncthreads();
        const int d = *s_pick;
        if (d < 0)
            return -1;
        want -= sh.res_digit;
        if (lv == 0)
            prefix = (uint32_t) d;
        else
            prefix = (prefix << 10) | (uint32_t) d;
        __syncthreads();
    }
    return (int) prefix;
}

/* The walk of sampler.c:270-299 (plus min-p) over n normalised probabilities without sorting
 * them. LIST = false: pn[] is a whole row in index order. LIST = true: pn[]/ids[] list, in any
 * order, every entry of the row up to some z bin; no entry outside the list has a pn whose bits
 * exceed `kout`, so the walk is exact as long as the kept prefix ends strictly above kout --
 * otherwise -1 is returned and the row is walked in full. */
/* `seen_max`: the largest key among the entries this thread has itself written to pn[] (the
 * threads together having written all of them), or SEEN_NONE to have the maximum looked for. */
constexpr uint32_t SEEN_NONE = 0xffffffffu;
template <bool LIST>
__device__ int sorted_descend(const float *pn, const uint32_t *ids, int n, float top_p, float min_p,
                              float u, uint32_t kout, SortedGenShared &sh, int *s_scan,
                              int *s_pick, uint32_t seen_max = SEEN_NONE) {
    const int  tid   = threadIdx.x;
    const bool use_p = top_p > 0.0f && top_p < 1.0f;
    const bool use_m = min_p > 0.0f;

    /* largest probability, then the min-p prefix: count and mass of pn >= min_p * pn_0 */
    uint32_t kmax = seen_max != SEEN_NONE ? seen_max : 0u;
    if (seen_max == SEEN_NONE)
        for_each_entry(pn, n, [&](int, float p) {
            const uint32_t key = __float_as_uint(p);
            kmax               = key > kmax ? key : kmax;
        });
    kmax = (uint32_t) block_max_u64((uint64_t) wave_max_u32(kmax), sh.red64);
    uint32_t n_m    = (uint32_t) n;
    uint64_t mass_m = 0;
    if (use_m) {
        const float floor_w = __fmul_rn(min_p, __uint_as_float(kmax));
        uint64_t    lm      = 0;
        uint64_t    lc      = 0;
        for_each_entry(pn, n, [&](int, float p) {
            if (p >= floor_w) {
                lm += pn_fx(p);
                ++lc;
            }
        });
        mass_m = block_sum_u64(lm, sh.red64);
        n_m    = (uint32_t) block_sum_u64(lc, sh.red64);
        if (n_m < 1u) { /* cannot happen (pn_0 >= min_p * pn_0 for min_p <= 1); keep the max */
            n_m    = 1u;
            mass_m = pn_fx(__uint_as_float(kmax));
        }
    }
    /* nucleus edge */
    bool     limited   = false;
    uint32_t edge_key  = 0u, edge_ties = 0u;
    uint64_t mass_keep = 0;
    uint32_t n_keep    = (uint32_t) n;
    bool     have_p    = false;
    if (use_p) {
        const uint64_t target = (uint64_t) __double2ull_ru((double) top_p * 0x1p62);
        uint32_t       kappa, cnt_above, ties;
        uint64_t       mass_above;
        if (sg_descent(pn, n, target, false, 0u, 0u, sh, kappa, cnt_above, mass_above, ties)) {
            const uint64_t each = pn_fx(__uint_as_float(kappa));
            uint64_t       j    = each ? (target - mass_above + each - 1) / each : 1;
            if (j < 1)
                j = 1;
            if (j > ties)
                j = ties;
            have_p    = true;
            limited   = true;
            edge_key  = kappa;
            edge_ties = (uint32_t) j;
            n_keep    = cnt_above + (uint32_t) j;
            mass_keep = mass_above + each * j;
        }
    }
    if (use_m && (!have_p || n_m < n_keep)) {
        /* the min-p prefix is the shorter one: every entry with pn >= floor, ties included */
        const float floor_w = __fmul_rn(min_p, __uint_as_float(kmax));
        if (LIST && __float_as_uint(floor_w) <= kout)
            return -1; /* entries outside the list may pass the floor too */
        limited   = true;
        n_keep    = n_m;
        mass_keep = mass_m;
        /* as an edge: keys >= floor, i.e. key > floor_bits - 1 with no ties taken from there */
        edge_key  = __float_as_uint(floor_w) ? __float_as_uint(floor_w) - 1u : 0u;
        edge_ties = 0u;
        if (__float_as_uint(floor_w) == 0u)
            limited = false;
    } else if (have_p) {
        if (LIST && edge_key <= kout)
            return -1; /* the nucleus may end among entries outside the list */
    } else {
        /* neither filter bites (top_p not reached by all n entries) */
        if (LIST)
            return -1;
        uint64_t lm = 0;
        for_each_entry(pn, n, [&](int, float p) { lm += pn_fx(p); });
        mass_keep = block_sum_u64(lm, sh.red64);
        limited   = false;
    }
    /* the draw: first entry of the kept prefix at which the running mass exceeds u * mass */
    /* running mass > u * mass  <=>  running mass >= floor(u * mass) + 1 in integers */
    const uint64_t target2 = (uint64_t) __double2ull_rd((double) u * (double) mass_keep) + 1ull;
    uint32_t       kd, cnt_above_d, ties_d;
    uint64_t       mass_above_d;
    int32_t        tok = -1;
    if (sg_descent(pn, n, target2, limited, edge_key, edge_ties, sh, kd, cnt_above_d,
                   mass_above_d, ties_d)) {
        const uint64_t each = pn_fx(__uint_as_float(kd));
        uint64_t       j    = each ? (target2 - mass_above_d + each - 1) / each : 1;
        if (j < 1)
            j = 1;
        if (j > ties_d)
            j = ties_d;
        if (LIST) {
            tok = list_jth_id(pn, ids, n, kd, (int) j, sh, s_scan, s_pick);
        } else if (j == 1) {
            /* the first entry (index order) with pn == kd */
            if (tid == 0)
                *s_pick = 0x7fffffff;
            __syncthreads();
            for_each_entry(pn, n, [&](int i, float p) {
                if (__float_as_uint(p) == kd)
                    atomicMin(s_pick, i);
            });
            __syncthreads();
            tok = *s_pick == 0x7fffffff ? -1 : *s_pick;
            __syncthreads();
        } else {
            /* the j-th entry (index order) with pn == kd: each thread takes a contiguous range */
            const int span = (n + TPB - 1) / TPB;
            const int lo   = tid * span < n ? tid * span : n;
            const int hi   = lo + span < n ? lo + span : n;
            int       mine = 0;
            {
                int i = lo; /* (eight loads in flight, as in for_each_entry) */
                for (; i + 8 <= hi; i += 8) {
                    float p[8];
#pragma unroll
                    for (int k = 0; k < 8; ++k)
                        p[k] = pn[i + k];
#pragma unroll
                    for (int k = 0; k < 8; ++k)
                        mine += __float_as_uint(p[k]) == kd;
                }
                for (; i < hi; ++i)
                    mine += __float_as_uint(pn[i]) == kd;
            }
            const int incl = block_scan_i32(mine, s_scan, nullptr);
            if (tid == 0)
                *s_pick = -1;
            __syncthreads();
            if (incl >= (int) j && incl - mine < (int) j) {
                int seen = incl - mine;
                for (int i = lo; i < hi; ++i) {
                    if (__float_as_uint(pn[i]) == kd && ++seen == (int) j) {
                        *s_pick = i;
                        break;
                    }
                }
            }
            __syncthreads();
            tok = *s_pick;
            __syncthreads();
        }
    }
    if (tok < 0 && !LIST) {
        /* not reachable with exact integer masses (the target never exceeds the kept mass);
         * kept as a defined outcome: the most probable entry */
        if (tid == 0)
            *s_pick = 0x7fffffff;
        __syncthreads();
        for_each_entry(pn, n, [&](int i, float p) {
            if (__float_as_uint(p) == kmax)
                atomicMin(s_pick, i);
        });
        __syncthreads();
        tok = *s_pick == 0x7fffffff ? 0 : *s_pick;
    }
    (void) n_keep;
    return tok;
}

/* The whole-row walk, for rows that neither the shortcut nor the list can serve (kept prefixes
 * of tens of thousands of entries, rows of equal values): the workgroup first writes the row's
 * normalised probabilities pn_i = (float)((double)p_i / sum) (sampler.c:246-253) into the probs
 * workspace, chunk by chunk, then walks them. Such rows are rare, so the row is not spread over
 * more workgroups. Called by every thread of a 256-thread workgroup. */
struct SortedRowArgs {
    float           inv_t;
    const uint64_t *chunk_best;
    const double   *chunk_sum;
    float          *probs;
    long            ld_probs;
};
template <int NV, bool PEN>
__device__ __forceinline__ int sorted_general_row(const RowView &rv, int row, int n_rows,
                                                  const SortedRowArgs &g, float top_p, float min_p,
                                                  float u, SortedGenShared &sh, uint32_t *s_cnt16,
                                                  uint64_t *s_tab, int *s_scan, int *s_pick,
                                                  double *s_total) {
    const int tid = threadIdx.x;
    __syncthreads(); /* the caller's use of the shared words is over */
    if (tid < 32)
        s_tab[tid] = g_expf_tab[tid];
    if (tid == 0) {
        double t = 0.0;
        for (int c = 0; c < rv.n_chunks; ++c)
            t += g.chunk_sum[(long) row * rv.n_chunks + c];
        *s_total = t;
    }
    const float  mx = key2f(best_key(row_best_from_chunks(g.chunk_best, row, rv.n_chunks, sh.red64)));
    const double tot = *s_total;
    float       *pn  = g.probs + (long) row * g.ld_probs;
    const float *rowp = rv.logits + (long) row * rv.ld;
    /* the next chunk's logits are asked for before this chunk is worked on */
    float4   v[NV], vnext[NV];
    uint32_t seen = 0u;
    {
        int base, end;
        chunk_bounds<NV>(rv, 0, base, end);
        load_raw<NV>(rv, rowp, base, end, v);
    }
    for (int chunk = 0; chunk < rv.n_chunks; ++chunk) {
        int base, end;
        chunk_bounds<NV>(rv, chunk, base, end);
        if (chunk + 1 < rv.n_chunks) {
            int nb, ne;
            chunk_bounds<NV>(rv, chunk + 1, nb, ne);
            load_raw<NV>(rv, rowp, nb, ne, vnext);
        }
        transform_loaded_chunk<NV, PEN>(rv, row, n_rows, base, end, s_cnt16, v);
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int e = base + 4 * (j * TPB + tid);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if (e + c < end) {
                    const float p = geist_expf_glibc_le0(softmax_arg(f4_get(v[j], c), mx, g.inv_t), s_tab);
                    const float q = (float) ((double) p / tot);
                    pn[e + c]     = q;
                    seen          = __float_as_uint(q) > seen ? __float_as_uint(q) : seen;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < NV; ++j)
            v[j] = vnext[j];
        __syncthreads(); /* the history table is rebuilt for the next chunk */
    }
    __threadfence_block();
    __syncthreads();
    return sorted_descend<false>(pn, nullptr, rv.n_vocab, top_p, min_p, u, 0u, sh, s_scan, s_pick,
                                 seen);
}

/* ============================================================================================
 * k_list_candidates: third pass over the rows flagged 1. Every element whose z bin is at or
 * before the row's bound is appended, in no particular order, to the row's list as (bits of its
 * normalised probability pn = (float)((double)p / sum), vocabulary id). A list longer than
 * CAND_CAP keeps counting; the row-final kernel then hands the row on.
 * ========================================================================================== */
constexpr int LIST_STAGE = 2048; /* candidates of one chunk staged in LDS */

template <int NV, bool PEN>
__global__ __launch_bounds__(TPB) void k_list_candidates(RowView rv, float inv_t,
                                                         const uint64_t *__restrict__ chunk_best,
                                                         const double *__restrict__ chunk_sum,
                                                         const int32_t *__restrict__ row_flag,
                                                         CandSpace cand) {
    static_assert(4 * NV <= 32, "one mask bit per element of a thread");
    __shared__ __align__(16) uint32_t s_cnt16[PEN ? NV * TPB * 2 : 1];
    __shared__ uint64_t s_red[NWAVES];
    __shared__ uint64_t s_tab[32];
    __shared__ double   s_total;
    __shared__ int      s_count, s_base;
    __shared__ float    s_arg[LIST_STAGE];
    __shared__ uint32_t s_id[LIST_STAGE];
    int                 row, chunk;
    xcd_row_chunk(row, chunk);
    const int tid = threadIdx.x;
    if (row_flag[row] != 1)
        return;
    if (tid < 32)
        s_tab[tid] = g_expf_tab[tid];
    if (tid == 0) {
        double t = 0.0;
        for (int c = 0; c < rv.n_chunks; ++c)
            t += chunk_sum[(long) row * rv.n_chunks + c];
        s_total = t;
        s_count = 0;
    }
    int base, end;
    chunk_bounds<NV>(rv, chunk, base, end);
    float4 v[NV];
    fetch_chunk<NV, PEN>(rv, row, (int) gridDim.y, base, end, s_cnt16, v);
    const float  mx  = key2f(best_key(row_best_from_chunks(chunk_best, row, rv.n_chunks, s_red)));
    const double tot = s_total;
    const int    B   = cand.row_bound[row];
    const float  thr = zbin_threshold(B); /* zbin(arg) <= B */
    uint32_t     mask = 0u;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int e = base + 4 * (j * TPB + tid);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const bool in = e + c < end && softmax_arg(f4_get(v[j], c), mx, inv_t) > thr;
            mask |= (uint32_t) in << (4 * j + c);
        }
    }
    /* places: inside the workgroup through LDS, one global add for the workgroup */
    int pos = wave_reserve(__popc(mask), &s_count);
    __syncthreads();
    const int n_blk = s_count;
    if (tid == 0)
        s_base = n_blk ? atomicAdd(&cand.count[(long) row * CAND_COUNT_STRIDE], n_blk) : 0;
    uint32_t *ck = cand.key + (long) row * CAND_CAP;
    uint32_t *ci = cand.idx + (long) row * CAND_CAP;
    if (n_blk <= LIST_STAGE) {
        /* stage (softmax argument, id) densely, then one exponential per staged entry */
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int e = base + 4 * (j * TPB + tid);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if ((mask >> (4 * j + c)) & 1u) {
                    s_arg[pos] = softmax_arg(f4_get(v[j], c), mx, inv_t);
                    s_id[pos]  = (uint32_t) (e + c);
                    ++pos;
                }
            }
        }
        __syncthreads();
        const int gbase = s_base;
        for (int i = tid; i < n_blk; i += TPB) {
            if (gbase + i < CAND_CAP) {
                const float p   = geist_expf_glibc_le0(s_arg[i], s_tab);
                ck[gbase + i]   = __float_as_uint((float) ((double) p / tot));
                ci[gbase + i]   = s_id[i];
            }
        }
    } else {
        __syncthreads();
        pos += s_base;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int e = base + 4 * (j * TPB + tid);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if ((mask >> (4 * j + c)) & 1u) {
                    if (pos < CAND_CAP) {
                        const float p =
                            geist_expf_glibc_le0(softmax_arg(f4_get(v[j], c), mx, inv_t), s_tab);
                        ck[pos] = __float_as_uint((float) ((double) p / tot));
                        ci[pos] = (uint32_t) (e + c);
                    }
                    ++pos;
                }
            }
        }
    }
}

/* ============================================================================================
 * list_walk_fast: the walk over a candidate list with ONE histogram. The keys that can matter lie
 * in (kout, kmax]; that range is cut into SG_BINS bins of equal width in key space, descending,
 * and the mass per bin is accumulated once (2^-62 fixed point, so exact and order-independent).
 * Prefix sums over the bins locate the bin in which the running mass of the sorted order reaches
 * a target; the handful of entries of that bin are ordered by counting and walked by one thread.
 * That is done for the nucleus edge (target top_p) and for the draw (target u * kept mass, bins
 * beyond the edge cut off), with the kept set described by one packed (key, id) threshold.
 * Returns the token, -1 when the list cannot certify the kept prefix (see sorted_descend), -2
 * when a bin holds more than TPB entries (long runs of equal values): the radix descent then
 * serves the list.
 * ========================================================================================== */
struct ListWalkShared {
    uint64_t mass[SG_BINS];
    uint64_t small[TPB];
    uint64_t srt[TPB];
    uint64_t red64[NWAVES];
    uint64_t scan64[NWAVES];
    uint64_t res_before, res_before_edge, out_pack, out_mass;
    int      res_bin, n_small;
};

__device__ __forceinline__ uint64_t wave_scan_u64(uint64_t v) {
    const int lane = threadIdx.x & (WAVE - 1);
#pragma unroll
    for (int d = 1; d < WAVE; d <<= 1) {
        const uint64_t o = ((uint64_t) (uint32_t) __shfl_up((int) (v >> 32), d, WAVE) << 32) |
                           (uint32_t) __shfl_up((int) (uint32_t) v, d, WAVE);
        if (lane >= d)
            v += o;
    }
    return v;
}

/* Orders and walks the entries of bin `b` that belong to the kept set (pack >= edge_pack): the
 * first one at which `before` plus the running mass reaches `target` goes to sh.out_pack, the
 * running mass including it to sh.out_mass. Returns false when the bin holds too many. */
__device__ __forceinline__ bool list_resolve_bin(const float *pn, const uint32_t *ids, int n, uint32_t kout,
                                 uint32_t kmax, int shift, int b, uint64_t before, uint64_t target,
                                 uint64_t edge_pack, ListWalkShared &sh) {
    const int tid = threadIdx.x;
    if (tid == 0)
        sh.n_small = 0;
    __syncthreads();
    for (int i0 = tid; i0 < n; i0 += 4 * TPB) {
        uint32_t k[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
            k[q] = i0 + q * TPB < n ? __float_as_uint(pn[i0 + q * TPB]) : 0u;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t key = k[q];
            if (key <= kout || (int) ((kmax - key) >> shift) != b)
                continue;
            const uint64_t pk = pack_best(key, ids[i0 + q * TPB]);
            if (pk < edge_pack)
                continue;
            const int at = atomicAdd(&sh.n_small, 1);
            if (at < TPB)
                sh.small[at] = pk;
        }
    }
    __syncthreads();
    const int c = sh.n_small;
    if (c > TPB)
        return false;
    if (tid < c) {
        const uint64_t me   = sh.small[tid];
        int            rank = 0;
        for (int j = 0; j < c; ++j)
            rank += sh.small[j] > me;
        sh.srt[rank] = me;
    }
    __syncthreads();
    if (tid < WAVE) { /* lane l walks entries 4l .. 4l+3 behind the lanes before it */
        uint64_t f[4], tot = 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int i = 4 * tid + q;
            f[q]        = i < c ? pn_fx(__uint_as_float(best_key(sh.srt[i]))) : 0ull;
            tot += f[q];
        }
        uint64_t run = before + wave_scan_u64(tot) - tot;
        int      at  = 0x7fffffff;
        uint64_t at_mass = 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            run += f[q];
            if (at == 0x7fffffff && 4 * tid + q < c && run >= target) {
                at      = 4 * tid + q;
                at_mass = run;
            }
        }
        const uint64_t hit = __ballot(at != 0x7fffffff);
        if (hit) {
            if (tid == __ffsll((long long) hit) - 1) {
                sh.out_pack = sh.srt[at];
                sh.out_mass = at_mass;
            }
        } else if (tid == (c > 0 ? (c - 1) / 4 : 0)) {
            /* not reached inside the bin (cannot happen with exact masses): its last entry */
            sh.out_pack = c > 0 ? sh.srt[c - 1] : 0ull;
            sh.out_mass = run;
        }
    }
    __syncthreads();
    return true;
}

__device__ __forceinline__ int list_walk_fast(const float *pn, const uint32_t *ids, int n,
                                              float top_p, float min_p, float u, uint32_t kout,
                                              ListWalkShared &sh) {
    const int  tid   = threadIdx.x;
    const bool use_p = top_p > 0.0f && top_p < 1.0f;
    const bool use_m = min_p > 0.0f;
    uint32_t   kmax  = 0u;
    for (int i0 = tid; i0 < n; i0 += 4 * TPB) {
        uint32_t k[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
            k[q] = i0 + q * TPB < n ? __float_as_uint(pn[i0 + q * TPB]) : 0u;
#pragma unroll
        for (int q = 0; q < 4; ++q)
            kmax = k[q] > kmax ? k[q] : kmax;
    }
    kmax = (uint32_t) block_max_u64((uint64_t) wave_max_u32(kmax), sh.red64);
    if (kmax <= kout)
        return -1;
    const int   bits    = 32 - __clz((int) (kmax - kout));
    const int   shift   = bits > 11 ? bits - 11 : 0;
    const float floor_w = __fmul_rn(min_p, __uint_as_float(kmax));
    for (int i = tid; i < SG_BINS; i += TPB)
        sh.mass[i] = 0ull;
    __syncthreads();
    uint64_t lm = 0;
    for (int i0 = tid; i0 < n; i0 += 4 * TPB) { /* the loads first: the adds below may alias them */
        float p4[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
            p4[q] = i0 + q * TPB < n ? pn[i0 + q * TPB] : 0.0f;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float    p   = p4[q];
            const uint32_t key = __float_as_uint(p);
            if (key <= kout) /* also the padding: kout >= 1 */
                continue;
            const uint64_t fx = pn_fx(p);
            atomicAdd((unsigned long long *) &sh.mass[(kmax - key) >> shift],
                      (unsigned long long) fx);
            if (use_m && p >= floor_w)
                lm += fx;
        }
    }
    __syncthreads();
    const uint64_t mass_m = use_m ? block_sum_u64(lm, sh.red64) : 0ull;
    /* exclusive prefix of the bins: thread t owns bins 8t .. 8t+7 */
    constexpr int PER = SG_BINS / TPB;
    uint64_t      own = 0;
#pragma unroll
    for (int q = 0; q < PER; ++q)
        own += sh.mass[tid * PER + q];
    uint64_t excl = wave_scan_u64(own);
    if ((tid & (WAVE - 1)) == WAVE - 1)
        sh.scan64[tid / WAVE] = excl;
    __syncthreads();
    for (int w = 0; w < tid / WAVE; ++w)
        excl += sh.scan64[w];
    excl -= own;
    /* the bin at which the running mass reaches `target`; optionally the mass before bin `be` */
    auto locate = [&](uint64_t target, int be) {
        if (tid == 0)
            sh.res_bin = -1;
        __syncthreads();
        uint64_t run = excl;
#pragma unroll
        for (int q = 0; q < PER; ++q) {
            const int      b = tid * PER + q;
            const uint64_t m = sh.mass[b];
            if (b == be)
                sh.res_before_edge = run;
            if (m && run < target && run + m >= target) {
                sh.res_bin    = b;
                sh.res_before = run;
            }
            run += m;
        }
        __syncthreads();
    };

    uint64_t edge_pack = 0ull, mass_keep = 0ull;
    bool     have_p    = false;
    if (use_p) {
        const uint64_t target = (uint64_t) __double2ull_ru((double) top_p * 0x1p62);
        locate(target, -1);
        const int b = sh.res_bin;
        if (b >= 0) {
            if (!list_resolve_bin(pn, ids, n, kout, kmax, shift, b, sh.res_before, target, 0ull, sh))
                return -2;
            have_p    = true;
            edge_pack = sh.out_pack;
            mass_keep = sh.out_mass;
        }
    }
    const uint32_t kf = __float_as_uint(floor_w);
    if (use_m && (!have_p || kf > best_key(edge_pack))) {
        if (kf <= kout)
            return -1; /* entries outside the list may pass the floor too */
        edge_pack = (uint64_t) kf << 32; /* every id with a key at or above the floor */
        mass_keep = mass_m;
    } else if (!have_p || best_key(edge_pack) <= kout) {
        return -1; /* the nucleus may reach past the list */
    }
    /* the draw: running mass > u * kept mass  <=>  running mass >= floor(u * kept mass) + 1 */
    const uint64_t target2 = (uint64_t) __double2ull_rd((double) u * (double) mass_keep) + 1ull;
    const int      be      = (int) ((kmax - best_key(edge_pack)) >> shift);
    locate(target2, be);
    int      bd     = sh.res_bin;
    uint64_t before = sh.res_before;
    if (bd < 0 || bd >= be) { /* inside the partly kept bin of the edge */
        bd     = be;
        before = sh.res_before_edge;
    }
    if (!list_resolve_bin(pn, ids, n, kout, kmax, shift, bd, before, target2, edge_pack, sh))
        return -2;
    return (int) best_idx(sh.out_pack);
}

/* k_sorted_candidates: one workgroup per row flagged 1 or 4 walks the row's list (staged in LDS
 * when it fits; flag 4: listed by the exp-sum pass, holding p). On success the flag is cleared; a row the list cannot serve -- too long, or a kept
 * prefix that may reach past the list -- takes the whole-row walk (flag 2).
 * direct_sum != NULL: every row was listed by the exp-sum pass under the min-p bound (the list
 * holds softmax arguments, not pn) and no other kernel ran in between: the row's sum is taken from the chunk
 * sums here (in chunk order, as everywhere), the bound on an unlisted element's pn from
 * direct_p_out = expf of the first z bin outside the list, and the flag is written for every
 * row.
 * walk_hint (page-locked host memory, or null): set to walk_call, the call's number, when a row
 * of the launch needs the whole-row walk -- the host then sends the next calls' such rows to
 * k_whole_row_coop, which spreads the walk over the row's chunks: this launch is told so by
 * defer_walk and only flags them 2. */
template <int NV, bool PEN>
__global__ __launch_bounds__(TPB) void k_sorted_candidates(RowView rv, SortedRowArgs g,
                                                           CandSpace cand, float top_p, float min_p,
                                                           const float *__restrict__ uniforms,
                                                           int32_t *__restrict__ row_flag,
                                                           int32_t *__restrict__ out,
                                                           const double *__restrict__ direct_sum,
                                                           int n_chunks, float direct_p_out,
                                                           int defer_walk,
                                                           uint32_t *__restrict__ walk_hint,
                                                           uint32_t walk_call) {
    extern __shared__ uint32_t s_key[]; /* CAND_CAP keys: every list is walked from LDS */
    __shared__ union {
        SortedGenShared gen;
        ListWalkShared  fast;
    } sh;
    __shared__ __align__(16) uint32_t s_cnt16[PEN ? NV * TPB * 2 : 1];
    __shared__ uint64_t s_tab[32];
    __shared__ double   s_total;
    __shared__ int      s_scan[NWAVES];
    __shared__ int      s_pick;
    __shared__ uint32_t s_idx[CAND_LDS];
    __shared__ double   s_csum[MAX_CHUNKS];
    const int row = blockIdx.x, tid = threadIdx.x;
    /* what the first steps need from memory is asked for at once, not one wait after the other:
     * the row's flag, the length of its list, the table of expf, the chunk sums (a thread each)
     * and the first two list entries of every thread (within the row's CAND_CAP places whatever
     * the length turns out to be) */
    const int       flag = direct_sum ? 5 : row_flag[row];
    const uint64_t  tabv = g_expf_tab[tid & 31];
    const int       n    = cand.count[(long) row * CAND_COUNT_STRIDE];
    const uint32_t *gk   = cand.key + (long) row * CAND_CAP;
    const uint32_t *gi   = cand.idx + (long) row * CAND_CAP;
    const double    csum = direct_sum && tid < n_chunks ? direct_sum[(long) row * n_chunks + tid] : 0.0;
    const float     u_row = uniforms[row];
    uint32_t        kpre[2];
#pragma unroll
    for (int q = 0; q < 2; ++q)
        kpre[q] = gk[q * TPB + tid];
    if (tid < 32)
        s_tab[tid] = tabv;
    if (tid < MAX_CHUNKS)
        s_csum[tid] = csum;
    __syncthreads();
    if (flag == 2) { /* sent past the list by the row-final kernel */
        if (tid == 0 && walk_hint)
            *walk_hint = walk_call;
        if (defer_walk)
            return; /* k_whole_row_coop follows and serves the rows flagged 2 */
        const int t = sorted_general_row<NV, PEN>(rv, row, rv.n_rows, g, top_p, min_p,
                                                  u_row, sh.gen, s_cnt16, s_tab, s_scan,
                                                  &s_pick, &s_total);
        if (tid == 0) {
            out[row]       = t;
            cand.path[row] = 3;
        }
        return;
    }
    if (flag != 1 && flag != 4 && flag != 5)
        return;
    int       tok = -1;
    double   sum  = 1.0;
    uint32_t kout = 0u;
    if (direct_sum) {
        /* every thread adds the chunk sums in chunk order */
        sum = 0.0;
        for (int c = 0; c < n_chunks; ++c)
            sum += s_csum[c];
        kout = __float_as_uint((float) ((double) direct_p_out / sum)) + 1u;
    } else {
        kout = cand.out_key[row];
        if (flag == 4)
            sum = cand.row_sum[row];
    }
    if (n >= 1 && n <= CAND_CAP) {
        /* flags 4, 5: the list holds the softmax arguments; p = expf(argument),
         * pn = (float)((double)p / sum), sampler.c:80, 251-253 */
#pragma unroll
        for (int q = 0; q < 2; ++q) { /* the entries asked for at the start */
            const int i = q * TPB + tid;
            if (i < n)
                s_key[i] = flag >= 4 ? __float_as_uint((float) ((double) geist_expf_glibc_le0(
                                                                    __uint_as_float(kpre[q]), s_tab) /
                                                                sum))
                                     : kpre[q];
        }
        for (int i0 = 2 * TPB; i0 < n; i0 += 8 * TPB) { /* eight independent loads in flight per thread */
            uint32_t k[8];
#pragma unroll
            for (int q = 0; q < 8; ++q)
                k[q] = i0 + q * TPB + tid < n ? gk[i0 + q * TPB + tid] : 0u;
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int i = i0 + q * TPB + tid;
                if (i < n)
                    s_key[i] = flag >= 4 ? __float_as_uint((float) ((double) geist_expf_glibc_le0(
                                                                        __uint_as_float(k[q]), s_tab) /
                                                                    sum))
                                         : k[q];
            }
        }
        if (n <= CAND_LDS) {
            for (int i = tid; i < n; i += TPB)
                s_idx[i] = gi[i];
            gi = s_idx;
        }
        __syncthreads();
        gk = s_key;
        const float *keys = reinterpret_cast<const float *>(gk);
        tok = list_walk_fast(keys, gi, n, top_p, min_p, u_row, kout, sh.fast);
        if (tok == -2) {
            __syncthreads();
            tok = sorted_descend<true>(keys, gi, n, top_p, min_p, u_row, kout, sh.gen,
                                       s_scan, &s_pick);
        }
    }
    /* what the list cannot certify takes the whole-row walk here and now (tok is the same in
     * every thread) */
    int path = 2;
    if (tok < 0) {
        if (tid == 0 && walk_hint)
            *walk_hint = walk_call;
        if (defer_walk) {
            if (tid == 0)
                row_flag[row] = 2;
            return;
        }
        tok  = sorted_general_row<NV, PEN>(rv, row, rv.n_rows, g, top_p, min_p, u_row,
                                           sh.gen, s_cnt16, s_tab, s_scan, &s_pick, &s_total);
        path = 3;
    }
    if (tid == 0) {
        row_flag[row]  = path == 3 ? 2 : 0;
        out[row]       = tok;
        cand.path[row] = path;
    }
}

} // namespace gs
#endif
