/*
 * sampler_kernels.hip -- the HIP kernels of the token-sampling path (gfx950).
 *
 * Kernel map (reference lines the arithmetic follows are cited at each kernel):
 *   k_tmax_scan      per-thread maxima (the single pass of the top-k path) and,
 *                    on request, the per-chunk maximum with its first index       sampler.c:52-62, 202-207
 *   k_scan_expsum    the one pass of the modes that weigh every element: per (row, chunk) the
 *                    maxima as above and the sum of expf((l - max) * inv_t); on request the
 *                    sums of the chunk's slabs, or the min-p candidates of the row
 *                                                                              sampler.c:52-62, 77-83
 *   k_final_argmax / _temperature / _topk / _sorted   per-row combine of each mode: argmax,
 *                    index-order CDF draw, top-k select + sorted softmax + top-p + min-p +
 *                    draw, top-p / min-p shortcut                             sampler.c:90-102, 209-222, 272-299
 *   k_topk_general   top-k for k above 128 and degenerate rows                 sampler.c:178-228
 *   k_cand_scan, k_final_cand (sampler_cands.h)   the top-k path for plain rows: the scan hands
 *                    each wavefront's leading groups on, the row-final kernel gathers nothing
 *                                                                              sampler.c:178-228
 *   k_list_candidates, k_sorted_candidates (sampler_sorted_prob.h)
 *                    full-vocabulary top-p / min-p for kept prefixes the shortcut cannot
 *                    serve: candidate list, then the whole row                 sampler.c:246-304
 *   k_write_probs    normalised probabilities of a row                        sampler.c:246-253
 *   k_chunk_lse, k_final_logprob   log-softmax of chosen tokens               tools/eval_geist.c:63-73
 *   k_penalties      in-place penalties                                       (no reference counterpart)
 *   k_spec_accept, k_spec_resid, k_spec_final (sampler_spec.h)
 *                    speculative-decode verification                          (no reference counterpart)
 *   k_rng_units      xorshift64* uniforms                                     sampler.c:35-48
 *
 * All streaming kernels use a (n_chunks, rows) grid of 256-thread workgroups and read each
 * logit exactly once per kernel; the logits are never written (k_penalties excepted).
 */
#include "sampler_kernels.h"

#include "sampler_device.h"

#include <cmath>
#include <type_traits>

namespace gs {

__device__ const uint64_t g_expf_tab[32] = GEIST_EXPF_TABLE_INIT;

/* Which (row, chunk) a workgroup of a (chunks, rows) grid works on. Workgroups go to the eight
 * XCDs round-robin by their linear id, and each XCD has its own L2. With the rows dealt out so
 * that every chunk of row r is handled on XCD r mod 8 -- in every pass, and the one-workgroup-
 * per-row kernels put row r there as well -- a later pass or the row-final kernel finds the
 * lines an earlier pass touched in the local L2. Needs a row count that is a multiple of 8. */
__device__ __forceinline__ void xcd_row_chunk(int &row, int &chunk) {
    row   = blockIdx.y;
    chunk = blockIdx.x;
    if ((gridDim.y & 7) == 0) {
        const int lin = blockIdx.y * gridDim.x + blockIdx.x, slot = lin >> 3;
        row           = (lin & 7) + 8 * (slot / (int) gridDim.x);
        chunk         = slot % (int) gridDim.x;
    }
}

template <int NV>
__device__ __forceinline__ void chunk_bounds(const RowView &rv, int chunk, int &base, int &end) {
    base = chunk * rv.per_chunk;
    end  = base + rv.per_chunk;
    if (end > rv.n_vocab)
        end = rv.n_vocab;
}

/* Loads and transforms the chunk [base, end) of a row; PEN selects the history lookup. `cnt16`
 * is an LDS table of NV*512 words when PEN, else unused. The logit loads are issued before the
 * history is read so that both are in flight together. */
/* The soft-cap maps the -inf that pads a partial chunk to -cap, a finite logit with weight in
 * every sum.  Positions at or beyond `end` are set back to -inf, so that consumers may keep
 * treating them as weightless without a bound test of their own.  (A -inf INSIDE the row does
 * become -cap, as it does in the reference: src/engine/sampler.c:95-99.) */
template <int NV>
__device__ __forceinline__ void remask_padding(const RowView &rv, int base, int end,
                                               float4 (&v)[NV]) {
    if (rv.softcap > 0.0f && end - base < NV * TPB * 4) {
        /* elements of this thread's first group that lie inside the row (<= 0: none). The empty
         * asm makes the value opaque: callers fetch inside loops, and the 4 * NV comparisons
         * would otherwise be hoisted out of them into as many scalar register pairs. */
        int lim = end - base - 4 * (int) threadIdx.x;
        asm volatile("" : "+v"(lim));
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int l = lim - 4 * j * TPB;
            v[j].x = l > 0 ? v[j].x : -INFINITY;
            v[j].y = l > 1 ? v[j].y : -INFINITY;
            v[j].z = l > 2 ? v[j].z : -INFINITY;
            v[j].w = l > 3 ? v[j].w : -INFINITY;
        }
    }
}

/* MASK = false compiles the allowed-token mask out (for callers that know rv.allowed is NULL and
 * are short of scalar registers). */
template <int NV, bool MASK = true>
__device__ __forceinline__ void mask_forbidden(const RowView &rv, int row, int base, int end,
                                               float4 (&v)[NV]) {
    if (MASK && rv.allowed) { /* forbidden tokens weigh nothing, whatever the transforms made */
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int e = base + 4 * (j * TPB + (int) threadIdx.x);
            if (e < end) {
                const uint32_t ok = allowed_nibble(rv, row, e);
                v[j].x = (ok & 1u) ? v[j].x : -INFINITY;
                v[j].y = (ok & 2u) ? v[j].y : -INFINITY;
                v[j].z = (ok & 4u) ? v[j].z : -INFINITY;
                v[j].w = (ok & 8u) ? v[j].w : -INFINITY;
            }
        }
    }
}
template <int NV, bool PEN, bool MASK = true>
__device__ __forceinline__ void fetch_chunk(const RowView &rv, int row, int n_rows, int base,
                                            int end, uint32_t *cnt16, float4 (&v)[NV]) {
    const float *rowp = rv.logits + (long) row * rv.ld;
    if (PEN) {
        const HistPrefetch pf = history_prefetch(rv, row, n_rows);
        load_raw<NV>(rv, rowp, base, end, v);
        history_clear<NV * TPB * 4>(cnt16);
        history_count(rv, row, pf, base, end, cnt16);
        apply_transform<NV>(rv, cnt16, v);
    } else {
        load_raw<NV>(rv, rowp, base, end, v);
        apply_transform<NV>(rv, nullptr, v);
    }
    remask_padding<NV>(rv, base, end, v);
    mask_forbidden<NV, MASK>(rv, row, base, end, v);
}
/* fetch_chunk() without its loads: `v` holds what load_raw() brought for the chunk. For a
 * caller that asks for the next chunk before it works on this one. */
template <int NV, bool PEN>
__device__ __forceinline__ void transform_loaded_chunk(const RowView &rv, int row, int n_rows,
                                                       int base, int end, uint32_t *cnt16,
                                                       float4 (&v)[NV]) {
    if (PEN) {
        const HistPrefetch pf = history_prefetch(rv, row, n_rows);
        history_clear<NV * TPB * 4>(cnt16);
        history_count(rv, row, pf, base, end, cnt16);
        apply_transform<NV>(rv, cnt16, v);
    } else {
        apply_transform<NV>(rv, nullptr, v);
    }
    remask_padding<NV>(rv, base, end, v);
    mask_forbidden<NV, true>(rv, row, base, end, v);
}

/* Row maximum from the per-chunk results; every thread returns the same packed value. */
__device__ __forceinline__ uint64_t row_best_from_chunks(const uint64_t *__restrict__ chunk_best,
                                                         int row, int n_chunks, uint64_t *s_red) {
    uint64_t b = 0;
    for (int c = threadIdx.x; c < n_chunks; c += TPB) {
        const uint64_t p = chunk_best[(long) row * n_chunks + c];
        b                = p > b ? p : b;
    }
    return block_max_u64(b, s_red);
}

/* ============================================================================================
 * k_scan_expsum: the one pass over the logits of the modes that weigh every element --
 * temperature, top-p / min-p, softmax, speculative verification. Per (row, chunk): the thread
 * maxima and the chunk's maximum with its first index (what k_tmax_scan writes;
 * sampler.c:52-62), then, once the row's maximum is known, the chunk's sum of
 * p_i = expf((l_i - max) * inv_t) in double (sampler.c:77-83); on request the sums of the
 * chunk's slabs, p at one token of the row (speculative verification needs p(x_j)), or the
 * row's min-p candidates.
 *
 * The row's maximum needs every chunk of the row, so the workgroups of a row meet half way
 * (row_best_meet): each keeps its chunk in registers, reports the chunk's maximum, waits for the
 * others' and sums the exponentials from the registers. The rows are read once.
 * ========================================================================================== */
/* The first index among a wavefront's elements whose key is `bk`, the wavefront's greatest,
 * packed with it; 0 when no element has that key (bk == 0: nothing but NaN). Every lane receives
 * it. Element c of group j of lane l sits at base + 4 (j TPB + tid) + c, so the first index is in
 * the first group that holds the value, there in the first lane, there in the first component:
 * a ballot per group instead of a search through each lane's elements and a reduction. Equal
 * keys are equal floats (f2key merges the zeros and gives every NaN key 0, which no float's
 * comparison matches). `bounded`: positions at or beyond `end` may hold anything. */
template <int NV, bool PLAIN>
__device__ __forceinline__ uint64_t wave_first_of(const float4 (&v)[NV], uint32_t bk, int base,
                                                  int end) {
    const float m   = key2f(bk);
    const int   tid = threadIdx.x;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int e = base + 4 * (j * TPB + tid);
        bool h0 = v[j].x == m, h1 = v[j].y == m, h2 = v[j].z == m, h3 = v[j].w == m;
        if (!PLAIN) {
            h0 = h0 && e < end;
            h1 = h1 && e + 1 < end;
            h2 = h2 && e + 2 < end;
            h3 = h3 && e + 3 < end;
        }
        const uint64_t hit = __builtin_amdgcn_ballot_w64(h0 || h1 || h2 || h3);
        if (hit) {
            const int lane = __builtin_ctzll(hit);
            const int c    = h0 ? 0 : h1 ? 1 : h2 ? 2 : 3;
            const int idx  = __builtin_amdgcn_readlane(e + c, lane);
            return pack_best(bk, (uint32_t) idx);
        }
    }
    return 0;
}

/* Where the thread maxima and the chunk results go, and the slots through which the workgroups
 * of a row meet. */
constexpr uint32_t SCAN_STAGE = 2048; /* candidates a workgroup stages in LDS */
struct FusedScan {
    float    *tmax;
    uint64_t *chunk_best;
    uint64_t *slots;
    uint32_t  wait_limit;
    uint32_t  local;    /* MeetSpace::local */
    uint64_t *s_red;    /* LDS, NWAVES words */
    uint64_t *s_bb;     /* LDS, one word */
    uint32_t *s_arrive; /* LDS, three arrival counters (and a fourth word), zero and published
                         * before use */
};

/* The row's maximum (packed with its first index) once every chunk of the row has reported its
 * own, for the workgroup that has just found `mine`. Every thread returns the same value.
 *
 * One wavefront of the workgroup (`reporter`: the one that combined the chunk's maximum) stores
 * `mine` (never zero) into the chunk's slot and polls the row's n_chunks <= 2 * WAVE slots, a
 * lane per slot, until none reads zero; the maximum of what it then holds is the row's, which
 * the other wavefronts receive through LDS behind a barrier. Stores and polls are device-scope
 * atomics (plain stores and loads, no read-modify-write: the slots of a row share a few cache
 * lines, and contended atomic updates of one line are what would make this wait slow), so no
 * fence is needed. An atomic of the caller's that the row's other workgroups must find
 * performed when they leave the wait has to have returned before the reporter gets here.
 *
 * A workgroup waits only for workgroups of its own row. The grid is dealt out so that a row's
 * workgroups have neighbouring ids and are started together; the wait is bounded all the same:
 * past `wait_limit` polls (0: at once) the workgroup stops waiting and finds the row's maximum
 * itself by reading the whole row, so every workgroup ends whatever the others do. */
/* A workgroup's word into its meeting slot: see MeetSpace::local. */
__device__ __forceinline__ void meet_store(uint64_t *slot, uint64_t v, uint32_t local) {
    if (local)
        *reinterpret_cast<volatile uint64_t *>(slot) = v;
    else
        __hip_atomic_store(slot, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <int NV, bool PEN>
__device__ __forceinline__ uint64_t row_best_meet(const RowView &rv, int row, int chunk,
                                                  int n_rows, uint64_t mine, bool reporter,
                                                  const FusedScan &fs, uint32_t *s_cnt16,
                                                  bool *met_out = nullptr) {
    static_assert(MAX_CHUNKS <= 2 * WAVE, "two slots per polling lane");
    const int tid = threadIdx.x, lane = tid & (WAVE - 1);
    const int C   = rv.n_chunks;
    uint64_t *row_slots = fs.slots + (long) row * C;
    if (reporter) { /* one wavefront, all its lanes */
        if (lane == 0)
            meet_store(row_slots + chunk, mine, fs.local);
        uint64_t a = 0, b = 0;
        uint32_t polls = 0;
        bool     met   = fs.wait_limit != 0;
        while (met) {
            a = lane < C ? __hip_atomic_load(row_slots + lane, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT)
                         : 0;
            b = lane + WAVE < C ? __hip_atomic_load(row_slots + lane + WAVE, __ATOMIC_RELAXED,
                                                    __HIP_MEMORY_SCOPE_AGENT)
                                : 0;
            const bool missing = (lane < C && a == 0) || (lane + WAVE < C && b == 0);
            if (__builtin_amdgcn_ballot_w64(missing) == 0)
                break;
            /* (no sleep between polls: a poll is a round trip to the second-level cache, during
             * which the wavefront issues nothing anyway; with one it is 0.4 us slower for one
             * row of 128256 and no faster for thousands of workgroups) */
            if (++polls > fs.wait_limit)
                met = false;
        }
        /* 1 is never a packed value: a row's first index is below 2^32 - 2 */
        const uint64_t got = met ? wave_max_u64(a > b ? a : b) : 1;
        if (lane == 0)
            *fs.s_bb = got;
    }
    __syncthreads();
    uint64_t bb = *fs.s_bb;
    if (met_out)
        *met_out = bb != 1;
    if (bb != 1)
        return bb;
    /* not met: the row's maximum from the row itself, 1024 elements at a time */
    bb = 0;
    for (int b0 = 0; b0 < rv.n_vocab; b0 += 4 * TPB) {
        const int e0 = b0 + 4 * TPB < rv.n_vocab ? b0 + 4 * TPB : rv.n_vocab;
        float4    w[1];
        fetch_chunk<1, PEN>(rv, row, n_rows, b0, e0, s_cnt16, w);
#pragma unroll
        for (int c = 3; c >= 0; --c) {
            const int e = b0 + 4 * tid + c;
            if (e < e0) {
                const uint64_t p = pack_best(f2key(f4_get(w[0], c)), (uint32_t) e);
                bb               = p > bb ? p : bb;
            }
        }
        __syncthreads(); /* the count table is rebuilt by the next round */
    }
    bb = block_max_u64(bb, fs.s_red);
    return bb ? bb : pack_best(0u, 0u);
}

/* expf(x) for x <= 0 from the hardware's 2^z, for the sums of the tolerance mode
 * (geist_hip_sampler_set_sums): x log2(e) as a binary32 product plus the product's rounding
 * error and the low part of log2(e), 2^z of the high part, one correction term. Relative error
 * about 1e-7 against the exact expf's half unit in the last place; -inf gives 0, NaN NaN. */
__device__ __forceinline__ float fast_expf_le0(float x) {
    const float L2E = 1.44269502f, L2E_LO = 1.92596299e-8f, LN2 = 0.693147182f;
    x               = x < -200.0f ? -200.0f : x; /* (2^z is 0 long before; keeps -inf out of the fma) */
    const float zh  = __fmul_rn(x, L2E);
    float       zl  = fmaf(x, L2E, -zh);
    zl              = fmaf(x, L2E_LO, zl);
    const float e   = __builtin_amdgcn_exp2f(zh);
    return fmaf(e, __fmul_rn(zl, LN2), e);
}

/* The work of one workgroup. PLAIN: a full, 16-byte aligned chunk without soft-cap or
 * allowed-token mask -- the common case, kept free of everything that would make the compiler
 * wait for all of the chunk's loads before the first group is looked at (a merge with the
 * element-wise loads of a ragged chunk, a branch around a mask load). */
/* NOMEET (tolerance mode, no penalties, no list): the workgroups of a row do not wait for one
 * another. Each sums its chunk against the chunk's own maximum, and a small launch behind the
 * pass (k_rescale_sums) scales every chunk's sums by expf((chunk maximum - row maximum) * inv_t)
 * -- exp((l - M) t) = exp((l - m) t) exp((m - M) t), which with arguments rounded to binary32
 * holds to a few 1e-7 relative: the tolerance mode's accuracy -- and evaluates p at the probed
 * token. What the two leave is what the meeting form leaves: chunk maxima, sums relative to the
 * row's maximum. (The scaling by the workgroup that arrives last at a counter of the row's,
 * inside the pass, was measured too: the acknowledged device-scope stores and the atomic it
 * needs keep every workgroup longer than the launch costs; 50.6 against 48.6 us for the
 * verification of 32 sequences, 53.3 with the meeting.) */
template <int NV, bool PEN, bool LISTM, bool SLABS, bool PLAIN, bool FAST, bool NOMEET>
__device__ __forceinline__ void expsum_chunk(const RowView &rv, int row, int chunk, int n_rows,
                                             int base, int end, float inv_t,
                                             double *__restrict__ chunk_sum,
                                             double *__restrict__ slab_sum,
                                             const int32_t *__restrict__ probe_token, int probe_L,
                                             float *__restrict__ probe_p, const CandSpace &list,
                                             int zb_list, uint32_t *s_cnt16, double *s_sum,
                                             uint64_t *s_tab, uint64_t tabv, double *s_tr,
                                             uint2 *s_stage, uint32_t *s_nstage,
                                             const FusedScan &fs) {
    const int tid = threadIdx.x;
    /* with penalties the work before the meet is long, and the row's other workgroups wait for
     * it: it is issued ahead of the exponentials of workgroups that have met */
    if (PEN)
        __builtin_amdgcn_s_setprio(3);
    /* Order of the loads: the probed token, the history, then the chunk. The groups of the
     * chunk are transformed one by one, each as soon as its own load has arrived: a barrier
     * with a full fence, or a transform over the whole chunk first, would keep the arithmetic
     * waiting for the last load. */
    /* spec verification: target row s*(L+1)+j is probed at draft token j of sequence s */
    int tok = -1;
    if (probe_token) {
        const int j = row % (probe_L + 1);
        if (j < probe_L)
            tok = probe_token[(long) (row / (probe_L + 1)) * probe_L + j];
    }
    HistPrefetch pf;
    if (PEN)
        pf = history_prefetch(rv, row, n_rows);
    float4       v[NV];
    const float *rowp = rv.logits + (long) row * rv.ld;
    if (PLAIN) {
        const float4 *p = reinterpret_cast<const float4 *>(rowp + base) + tid;
        if (rv.stream_loads) {
#pragma unroll
            for (int j = 0; j < NV; ++j)
                v[j] = load_streaming(p + j * TPB);
        } else {
#pragma unroll
            for (int j = 0; j < NV; ++j)
                v[j] = p[j * TPB];
        }
    } else {
        load_raw<NV>(rv, rowp, base, end, v);
    }
    if (tid < 32)
        s_tab[tid] = tabv;
    if (tid < 4) /* three arrival counters and the staging list's length */
        fs.s_arrive[tid] = 0;
    if (PEN) {
        history_clear<NV * TPB * 4>(s_cnt16);
        history_count(rv, row, pf, base, end, s_cnt16);
    } else {
        lds_barrier(); /* publishes s_tab (the history's barriers do when PEN) */
    }
    uint64_t bb;
    {
        /* first half of the one pass: transform each group as its load arrives, keep the
         * thread's maximum (k_tmax_scan's output) and the chunk's (sampler.c:52-62), then meet
         * the row's other chunks */
        float tm = -__builtin_inff();
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            transform_group<PEN, !PLAIN>(rv, row, s_cnt16, 4 * (j * TPB + tid), base, end, v[j]);
            tm = max3f(tm, max3f(v[j].x, v[j].y, v[j].z), v[j].w);
        }
        if (base + 4 * tid >= end)
            tm = __builtin_nanf("");
        if (fs.tmax) /* (wanted by the row-final kernel of the top-p path only) */
            fs.tmax[((long) row * rv.n_chunks + chunk) * TPB + tid] = tm;
        /* the wavefront's best, then the chunk's: each wavefront deposits its own in LDS and
         * the one that arrives last (no barrier: the others need not wait for it) combines
         * them, reports the chunk's and waits for the row's */
        const uint32_t bk   = wave_max_u32(f2key(tm));
        uint64_t       best = wave_first_of<NV, PLAIN>(v, bk, base, end);
        uint32_t prior = 0;
        if (LISTM && chunk == 0 && tid == 0) /* the list the second half appends to starts empty */
            prior = (uint32_t) atomicExch(&list.count[(long) row * CAND_COUNT_STRIDE], 0);
        if ((tid & (WAVE - 1)) == 0) {
            /* `prior` an operand of the deposit: the exchange above has returned before this
             * wavefront arrives, so before the chunk's slot is stored */
            asm volatile("" : "+v"(best) : "v"(prior));
            fs.s_red[tid / WAVE] = best;
        }
        const bool last = wave_arrives_last(fs.s_arrive);
        if (last) {
            best = fs.s_red[0];
#pragma unroll
            for (int w = 1; w < NWAVES; ++w)
                best = fs.s_red[w] > best ? fs.s_red[w] : best;
            if (!best) /* an all-NaN chunk reports key 0 at its first index */
                best = pack_best(0u, (uint32_t) base);
            if ((tid & (WAVE - 1)) == 0)
                fs.chunk_best[(long) row * rv.n_chunks + chunk] = best;
        }
        if (NOMEET) {
            if (last && (tid & (WAVE - 1)) == 0)
                *fs.s_bb = best; /* the chunk's own */
            lds_barrier();
            bb = *fs.s_bb;
        } else {
            bb = row_best_meet<NV, PEN>(rv, row, chunk, n_rows, best, last, fs, s_cnt16);
        }
    }
    if (PEN)
        __builtin_amdgcn_s_setprio(0);
    float mx = key2f(best_key(bb));
    /* (NOMEET: a chunk of nothing but -inf is summed against 0, so that it weighs 0 and not
     * NaN; the scaling by the row's maximum makes the row's sums NaN where the meeting form's
     * are, in a row of nothing but -inf) */
    if (NOMEET && mx == -__builtin_inff())
        mx = 0.0f;

    if (!NOMEET && tok >= base && tok < end) {
        /* the thread that holds the probed element evaluates it by itself (before the sums, so
         * that each group's registers are free once it has been added up) */
        const int off = tok - base, f = off >> 2;
        if ((f & (TPB - 1)) == tid) {
            const int j = f / TPB;
            float     x = 0.0f;
#pragma unroll
            for (int jj = 0; jj < NV; ++jj)
                if (jj == j)
                    x = f4_get(v[jj], off & 3);
            probe_p[row] = geist_expf_glibc_le0(softmax_arg(x, mx, inv_t), s_tab);
        }
    }
    /* SLABS with eight groups: a group's sum goes straight into the table through which the
     * wavefront's eight sums are transposed (below), so no sum stays in a register */
    constexpr bool TRANSPOSED = SLABS && NV == 8;
    volatile double *tr = s_tr + (tid / WAVE) * (8 * WAVE);
    double      acc  = 0.0;
    double      accs[SLABS && !TRANSPOSED ? NV : 1];
    const float list_thr = zbin_threshold(zb_list); /* zbin(arg) <= zb_list */
    /* positions at or beyond `end` hold -inf (load_raw): they weigh exactly 0 and land in no
     * bin, so the loop carries no bound tests */
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        double a4;
        float  args[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            args[c]        = softmax_arg(f4_get(v[j], c), mx, inv_t);
            const double p = (double) (FAST ? fast_expf_le0(args[c])
                                            : geist_expf_glibc_le0(args[c], s_tab));
            a4             = c == 0 ? p : a4 + p;
        }
        if (LISTM) {
            /* the group's candidates go to the workgroup's staging list in LDS right away (the
             * softmax argument and the id; the list walk takes the exponential of the few
             * hundred entries it reads), so that the group's registers are free afterwards */
            const bool c0 = args[0] > list_thr, c1 = args[1] > list_thr, c2 = args[2] > list_thr,
                       c3 = args[3] > list_thr;
            if (__builtin_amdgcn_ballot_w64(c0 || c1 || c2 || c3)) {
                const int e = base + 4 * (j * TPB + tid);
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    if (c == 0 ? c0 : c == 1 ? c1 : c == 2 ? c2 : c3) {
                        const uint32_t at = __hip_atomic_fetch_add(
                            s_nstage, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                        if (at < SCAN_STAGE)
                            s_stage[at] = make_uint2(__float_as_uint(args[c]), (uint32_t) (e + c));
                    }
                }
            }
        }
        if (TRANSPOSED)
            tr[j * WAVE + ((tid & (WAVE - 1)) ^ j)] = a4;
        else if (SLABS)
            accs[j] = a4;
        else
            acc += a4;
        /* four evaluations in flight are enough to cover the latencies; left alone, the
         * compiler interleaves all 4 * NV of them and the registers that takes cost most of the
         * occupancy. The empty asm ties the next group's inputs to this group's sum. */
        if (j + 1 < NV) {
            if (TRANSPOSED)
                asm volatile("" : "+v"(a4), "+v"(v[j + 1].x), "+v"(v[j + 1].y),
                                  "+v"(v[j + 1].z), "+v"(v[j + 1].w));
            else if (SLABS)
                asm volatile("" : "+v"(accs[j]), "+v"(v[j + 1].x), "+v"(v[j + 1].y),
                                  "+v"(v[j + 1].z), "+v"(v[j + 1].w));
            else
                asm volatile("" : "+v"(acc), "+v"(v[j + 1].x), "+v"(v[j + 1].y),
                                  "+v"(v[j + 1].z), "+v"(v[j + 1].w));
        }
    }
    /* The chunk's sums: wavefront totals (lane 63 of the DPP scan) deposited in LDS, combined by
     * the wavefront that arrives last, in the order wavefront 0..3 (and slab 0..NV-1 for the
     * chunk's sum, which is the sum of its slab sums). No barrier: a wavefront that is done
     * leaves. */
    {
        const int  lane = tid & (WAVE - 1), w = tid / WAVE;
        const long at   = (long) row * rv.n_chunks + chunk;
        if (TRANSPOSED) {
            /* eight sums over the wavefront at once, through LDS: sum j of lane l went to place
             * [j][l] of the wavefront's 8 x 64 table, now lane l adds the eight entries
             * [l / 8][8 (l % 8) ..] in order and three DPP steps add up the eight lanes of a
             * group: lane 8 j + 7 ends with sum j. (Eight DPP reductions one after the other
             * took as long as a third of the exponentials.) Places are swizzled by the row
             * number, so that the lanes of a read hit different banks. */
            const int g = lane >> 3, first = 8 * (lane & 7);
            double    r = tr[g * WAVE + (first ^ g)];
#pragma unroll
            for (int i = 1; i < 8; ++i)
                r += tr[g * WAVE + ((first + i) ^ g)];
            r += dpp_fetch_f64<0x111, 0xf>(r); /* row_shr:1, 2, 4: the lane and the seven */
            r += dpp_fetch_f64<0x112, 0xf>(r); /* before it                               */
            r += dpp_fetch_f64<0x114, 0xf>(r);
            if ((lane & 7) == 7)
                s_sum[w * NV + g] = r;
        } else if (SLABS) {
#pragma unroll
            for (int j = 0; j < NV; ++j) {
                const double t = wave_scan_f64_dpp(accs[TRANSPOSED ? 0 : j]);
                if (lane == WAVE - 1)
                    s_sum[w * NV + j] = t;
            }
        } else {
            const double t = wave_scan_f64_dpp(acc);
            if (lane == WAVE - 1)
                s_sum[w] = t;
        }
        if (wave_arrives_last(fs.s_arrive + 1) && lane == 0) {
            constexpr int NS = SLABS ? NV : 1;
            double        total = 0.0;
#pragma unroll
            for (int j = 0; j < NS; ++j) {
                double r = s_sum[j];
#pragma unroll
                for (int x = 1; x < NWAVES; ++x)
                    r += s_sum[x * NS + j];
                if (SLABS)
                    slab_sum[at * SLABS_MAX + j] = r;
                total += r;
            }
            chunk_sum[at] = total;
        }
    }
    if (LISTM) {
        /* the wavefront that arrives last moves the staged entries to the row's list: one add to
         * the row's counter per workgroup. A workgroup with more candidates than the staging
         * list holds reports more than the row's list can hold, which sends the row to the
         * whole-row walk. */
        if (wave_arrives_last(fs.s_arrive + 2)) {
            const int      lane  = tid & (WAVE - 1);
            const uint32_t n     = *s_nstage;
            const uint32_t total = n > SCAN_STAGE ? (uint32_t) CAND_CAP + 1u : n;
            int            at    = 0;
            if (lane == 0 && total)
                at = atomicAdd(&list.count[(long) row * CAND_COUNT_STRIDE], (int) total);
            at = __builtin_amdgcn_readfirstlane(at);
            uint32_t *ck = list.key + (long) row * CAND_CAP;
            uint32_t *ci = list.idx + (long) row * CAND_CAP;
            for (uint32_t i = lane; i < n && i < SCAN_STAGE; i += WAVE) {
                const uint2 t = s_stage[i];
                if (at + (int) i < CAND_CAP) {
                    ck[at + i] = t.x;
                    ci[at + i] = t.y;
                }
            }
        }
    }
}

/* The penalised list-making form needs 82 registers when left alone, two more than let a sixth
 * workgroup share a compute unit; held to 80 it spills nothing and a launch of 128 x 151936 is
 * about a microsecond shorter. (Held to 72 or 64 it spills and is slower.) */
template <int NV, bool PEN, bool LISTM, bool SLABS, bool FAST = false, bool NOMEET = false>
__global__ __launch_bounds__(TPB, (NV == 8 && PEN && LISTM) ? 6 : 1) void k_scan_expsum(RowView rv, float inv_t,
                                                     float *__restrict__ tmax,
                                                     uint64_t *__restrict__ chunk_best,
                                                     double *__restrict__ chunk_sum,
                                                     double *__restrict__ slab_sum,
                                                     const int32_t *__restrict__ probe_token,
                                                     int probe_L, float *__restrict__ probe_p,
                                                     CandSpace list, int zb_list, MeetSpace meet) {
    
    __shared__ __align__(16) uint32_t s_cnt16[PEN ? NV * TPB * 2 : 1];
    __shared__ double   s_sum[SLABS ? NWAVES * NV : NWAVES];
    __shared__ uint64_t s_tab[32];
    __shared__ uint64_t s_red[NWAVES], s_bb;
    __shared__ uint32_t s_arrive[4];
    /* the staging list of the candidates: in the history's count table when there is one */
    __shared__ uint2 s_stage_own[(LISTM && !PEN) ? SCAN_STAGE : 1];
    static_assert(!(LISTM && PEN) || sizeof(s_cnt16) >= SCAN_STAGE * sizeof(uint2),
                  "the count table holds the staging list");
    uint2 *s_stage = PEN ? reinterpret_cast<uint2 *>(s_cnt16) : s_stage_own;
    /* the table the slab sums are transposed through: the history's count table has the size
     * and is free once the row's workgroups have met */
    __shared__ __align__(16) double s_tr_own[(SLABS && NV == 8 && !PEN) ? NWAVES * 8 * WAVE : 1];
    static_assert(!(SLABS && NV == 8 && PEN) || sizeof(s_cnt16) >= NWAVES * 8 * WAVE * sizeof(double),
                  "the count table holds the transposed sums");
    double *s_tr = PEN ? reinterpret_cast<double *>(s_cnt16) : s_tr_own;
    const int tid = threadIdx.x;
    int       row, chunk;
    xcd_row_chunk(row, chunk);
    /* the table's words are asked for here and put into LDS after the chunk's loads have been
     * issued: written at once, the wait for them would stand before those loads */
    const uint64_t tabv = g_expf_tab[tid & 31];
    /* the slots that the launch before this one used, back to zero for the launch after */
    {
        const uint32_t wg = blockIdx.y * gridDim.x + blockIdx.x, n_wg = gridDim.x * gridDim.y;
        for (uint32_t i = wg * TPB + tid; i < meet.stale_count; i += n_wg * TPB)
            meet.stale[i] = 0;
    }
    int base, end;
    chunk_bounds<NV>(rv, chunk, base, end);
    FusedScan fs;
    fs.tmax       = tmax;
    fs.chunk_best = chunk_best;
    fs.slots      = meet.slots;
    fs.wait_limit = meet.wait_limit;
    fs.local      = meet.local;
    fs.s_red      = s_red;
    fs.s_bb       = &s_bb;
    fs.s_arrive   = s_arrive;
    static_assert(!NOMEET || (FAST && !PEN && !LISTM), "the form without a meeting");
    const bool plain = rv.vec_ok && end - base == NV * TPB * 4 && !(rv.softcap > 0.0f) &&
                       rv.allowed == nullptr;
    if (plain)
        expsum_chunk<NV, PEN, LISTM, SLABS, true, FAST, NOMEET>(
            rv, row, chunk, (int) gridDim.y, base, end, inv_t, chunk_sum, slab_sum,
            probe_token, probe_L, probe_p, list, zb_list, s_cnt16, s_sum, s_tab, tabv, s_tr, s_stage,
            s_arrive + 3, fs);
    else
        expsum_chunk<NV, PEN, LISTM, SLABS, false, FAST, NOMEET>(
            rv, row, chunk, (int) gridDim.y, base, end, inv_t, chunk_sum, slab_sum,
            probe_token, probe_L, probe_p, list, zb_list, s_cnt16, s_sum, s_tab, tabv, s_tr, s_stage,
            s_arrive + 3, fs);
}

/* The scaling of the form without a meeting: a wavefront per row, a lane per chunk. */
template <bool SLABS>
__global__ __launch_bounds__(WAVE) void k_rescale_sums(RowView rv, float inv_t,
                                                      const uint64_t *__restrict__ chunk_best,
                                                      double *__restrict__ chunk_sum,
                                                      double *__restrict__ slab_sum,
                                                      const int32_t *__restrict__ probe_token,
                                                      int probe_L, float *__restrict__ probe_p) {
    __shared__ uint64_t s_tab[32];
    const int row = blockIdx.x, lane = threadIdx.x, C = rv.n_chunks;
    if (lane < 32)
        s_tab[lane] = g_expf_tab[lane];
    const long r0 = (long) row * C;
    uint64_t   ba = lane < C ? chunk_best[r0 + lane] : 0, bb2 = lane + WAVE < C ? chunk_best[r0 + lane + WAVE] : 0;
    int        tok = -1;
    if (probe_token && lane == 0) {
        const int j = row % (probe_L + 1);
        if (j < probe_L)
            tok = probe_token[(long) (row / (probe_L + 1)) * probe_L + j];
    }
    float x_tok = 0.0f;
    if (tok >= 0)
        x_tok = rv.logits[(long) row * rv.ld + tok];
    __syncthreads();
    const uint64_t rowb = wave_max_u64(ba > bb2 ? ba : bb2);
    const float    M    = key2f(best_key(rowb));
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int c = lane + h * WAVE;
        if (c >= C)
            continue;
        const float  mc = key2f(best_key(h ? bb2 : ba));
        const double f  = (double) geist_expf_glibc_le0(softmax_arg(mc, M, inv_t), s_tab);
        chunk_sum[r0 + c] *= f;
        if (SLABS) {
            double v8[SLABS_MAX];
#pragma unroll
            for (int j = 0; j < SLABS_MAX; ++j)
                v8[j] = slab_sum[(r0 + c) * SLABS_MAX + j];
#pragma unroll
            for (int j = 0; j < SLABS_MAX; ++j)
                slab_sum[(r0 + c) * SLABS_MAX + j] = v8[j] * f;
        }
    }
    if (tok >= 0)
        probe_p[row] = geist_expf_glibc_le0(softmax_arg(x_tok, M, inv_t), s_tab);
}

/* ============================================================================================
 * k_tmax_scan: the one pass over the logits of the top-k path. Each thread keeps only the
 * maximum of the 4*NV elements it read (after penalties and soft-cap) and stores it; nothing
 * else leaves the workgroup. The row-final kernel picks the k-th largest of a row's thread
 * maxima -- a lower bound of the row's k-th largest element, because k different threads hold
 * an element at or above it -- and re-reads only the elements of the threads at or above that
 * bound (about k of them, 4*NV elements each).
 * max ignores NaN; a thread with no element of the row stores NaN and is never chosen.
 * ========================================================================================== */
template <int NV, bool PEN, bool BEST>
__global__ __launch_bounds__(TPB) void k_tmax_scan(RowView rv, float *__restrict__ tmax,
                                                   uint64_t *__restrict__ chunk_best,
                                                   int32_t *__restrict__ zero_per_row) {
    __shared__ __align__(16) uint32_t s_cnt16[PEN ? NV * TPB * 2 : 1];
    __shared__ uint64_t s_red[NWAVES];
    int row, chunk;
    xcd_row_chunk(row, chunk);
    const int tid = threadIdx.x;
    if (BEST && zero_per_row && chunk == 0 && tid == 0)
        zero_per_row[row] = 0; /* a counter the following pass adds to */
    int       base, end;
    chunk_bounds<NV>(rv, chunk, base, end);
    float4 v[NV];
    float  tm = -__builtin_inff();
    if (PEN && rv.vec_ok && end - base == NV * TPB * 4 && !(rv.softcap > 0.0f) &&
        rv.allowed == nullptr) {
        /* the common case with penalties: each group is penalised as soon as its own load has
         * arrived, while the later ones are still in flight (fetch_chunk() transforms the chunk
         * as a whole, after its last load) */
        const HistPrefetch pf = history_prefetch(rv, row, (int) gridDim.y);
        const float4      *p =
            reinterpret_cast<const float4 *>(rv.logits + (long) row * rv.ld + base) + tid;
#pragma unroll
        for (int j = 0; j < NV; ++j)
            v[j] = p[j * TPB];
        history_clear<NV * TPB * 4>(s_cnt16);
        history_count(rv, row, pf, base, end, s_cnt16);
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            transform_group<PEN, false>(rv, row, s_cnt16, 4 * (j * TPB + tid), base, end, v[j]);
            tm = max3f(tm, max3f(v[j].x, v[j].y, v[j].z), v[j].w);
        }
    } else {
        fetch_chunk<NV, PEN>(rv, row, (int) gridDim.y, base, end, s_cnt16, v);
#pragma unroll
        for (int j = 0; j < NV; ++j)
            tm = max3f(tm, max3f(v[j].x, v[j].y, v[j].z), v[j].w);
    }
    if (base + 4 * tid >= end)
        tm = __builtin_nanf("");
    tmax[((long) row * rv.n_chunks + chunk) * TPB + tid] = tm;
    if (BEST) {
        /* the chunk's maximum and the first index holding it (sampler.c:52-62): only threads
         * whose own maximum equals the chunk's look for the index */
        const uint32_t mykey = f2key(tm);
        uint32_t       bk    = wave_max_u32(mykey);
        bk = (uint32_t) (block_max_u64((uint64_t) bk, s_red));
        uint64_t best = 0;
        if (mykey == bk) {
            int first = 0x7fffffff;
#pragma unroll
            for (int j = NV - 1; j >= 0; --j) {
                const int e = base + 4 * (j * TPB + tid);
#pragma unroll
                for (int c = 3; c >= 0; --c)
                    if (e + c < end && f2key(f4_get(v[j], c)) == bk)
                        first = e + c;
            }
            if (first != 0x7fffffff)
                best = pack_best(bk, (uint32_t) first);
        }
        best = block_max_u64(best, s_red);
        if (tid == 0) /* an all-NaN chunk reports key 0 at its first index */
            chunk_best[(long) row * rv.n_chunks + chunk] =
                best ? best : pack_best(0u, (uint32_t) base);
    }
}

/* ============================================================================================
 * finish_sorted: the tail every sorted mode shares. `spack` holds n survivors in walk order
 * (key descending, index ascending), packed as pack_best(). Computes, as the reference does on
 * its sorted array: p_i = expf((l_i - l_0) * inv_t) (sampler.c:219 via 68-85), optionally
 * pn_i = (float)((double)p_i / sum) (sampler.c:251-253), the nucleus (sampler.c:273-283), the
 * min-p prefix, and the draw u * mass walked in order (sampler.c:290-299 / 90-102).
 * Each thread owns a run of consecutive entries; prefix sums are per-thread sequential sums
 * combined by a workgroup scan. Weights are recomputed on each walk instead of being stored.
 * Returns the chosen vocabulary id to every thread.
 * ========================================================================================== */
struct FinishShared {
    double   scan[NWAVES];
    double   mass;
    float    w0;
    int      n_p;
    int      n_m;
    int      pick;
    uint64_t tab[32];
};

__device__ int finish_sorted(int n, const uint64_t *spack, float inv_t, float top_p, float min_p,
                             float u, FinishShared &fs) {
    const int  tid   = threadIdx.x;
    const bool use_p = top_p > 0.0f && top_p < 1.0f;
    const bool use_m = min_p > 0.0f;
    const bool norm  = use_p || use_m;
    const int  ipt   = (n + TPB - 1) / TPB;
    const int  lo    = tid * ipt < n ? tid * ipt : n;
    const int  hi    = lo + ipt < n ? lo + ipt : n;

    if (tid < 32)
        fs.tab[tid] = g_expf_tab[tid];
    if (tid == 0) {
        fs.n_p  = n;
        fs.n_m  = 0;
        fs.pick = 0x7fffffff;
    }
    __syncthreads();
    const float l0 = key2f(best_key(spack[0]));
#define GS_P(i) geist_expf_glibc_le0(softmax_arg(key2f(best_key(spack[i])), l0, inv_t), fs.tab)

    double part = 0.0;
    for (int i = lo; i < hi; ++i)
        part += (double) GS_P(i);
    double sum;
    double incl = block_scan_f64(part, fs.scan, &sum);
#define GS_W(i) (norm ? (float) ((double) GS_P(i) / sum) : GS_P(i))
    if (norm) {
        part = 0.0;
        for (int i = lo; i < hi; ++i)
            part += (double) GS_W(i);
        incl = block_scan_f64(part, fs.scan, nullptr);
    }
    const double off = incl - part; /* exclusive prefix of this thread's entries */

    int keep = n;
    if (norm) {
        if (tid == 0)
            fs.w0 = GS_W(0);
        __syncthreads();
        const float floor_w = __fmul_rn(min_p, fs.w0);
        double      run     = off;
        int         cnt_m   = 0;
        int         first_p = 0x7fffffff;
        for (int i = lo; i < hi; ++i) {
            const float w = GS_W(i);
            run += (double) w;
            if (use_p && first_p == 0x7fffffff && run >= (double) top_p)
                first_p = i + 1;
            if (use_m && w >= floor_w)
                ++cnt_m;
        }
        /* one atomic per wavefront: every thread past the nucleus' end has a position to
         * report, and that many atomics on one word of LDS take microseconds */
        {
            const uint32_t fp = ~wave_max_u32(~(uint32_t) first_p);
            const int      wave_m =
                __builtin_amdgcn_readlane(wave_scan_i32_dpp(cnt_m), WAVE - 1);
            if ((tid & (WAVE - 1)) == 0) {
                if (use_p && fp != 0x7fffffffu)
                    atomicMin(&fs.n_p, (int) fp);
                if (use_m && wave_m)
                    atomicAdd(&fs.n_m, wave_m);
            }
        }
        __syncthreads();
        keep = fs.n_p;
        if (use_m) {
            const int m = fs.n_m < 1 ? 1 : fs.n_m;
            keep        = m < keep ? m : keep;
        }
        if (keep < 1)
            keep = 1;
    }

    /* mass = inclusive prefix at entry keep-1 */
    if (keep - 1 >= lo && keep - 1 < hi) {
        double run = off;
        for (int i = lo; i <= keep - 1; ++i)
            run += (double) GS_W(i);
        fs.mass = run;
    }
    __syncthreads();
    const double target = (double) u * fs.mass;
    {
        double   run  = off;
        uint32_t mine = 0x7fffffffu;
        for (int i = lo; i < hi && i < keep; ++i) {
            run += (double) GS_W(i);
            if (target < run) {
                mine = (uint32_t) i;
                break;
            }
        }
        mine = ~wave_max_u32(~mine); /* (as above: one atomic per wavefront) */
        if ((tid & (WAVE - 1)) == 0 && mine != 0x7fffffffu)
            atomicMin(&fs.pick, (int) mine);
    }
    __syncthreads();
#undef GS_P
#undef GS_W
    const int at = fs.pick == 0x7fffffff ? keep - 1 : fs.pick;
    return (int) best_idx(spack[at]);
}

/* finish_sorted for n <= 64 * IPT survivors on ONE wavefront (call with all 64 lanes of a
 * single wave): lane l owns entries IPT*l .. IPT*l + IPT-1, the prefix sums are wavefront scans,
 * no barrier. `tab` is the expf table in LDS. */
template <int IPT>
__device__ int finish_sorted_wave(int n, const uint64_t *spack, float inv_t, float top_p,
                                  float min_p, float u, const uint64_t *tab) {
    const int   lane  = threadIdx.x & (WAVE - 1);
    const bool  use_p = top_p > 0.0f && top_p < 1.0f;
    const bool  use_m = min_p > 0.0f;
    const bool  norm  = use_p || use_m;
    const float l0    = key2f(best_key(spack[0]));
    float       w[IPT];
    double      part = 0.0;
#pragma unroll
    for (int t = 0; t < IPT; ++t) {
        const int i = IPT * lane + t;
        w[t] = i < n ? geist_expf_glibc_le0(softmax_arg(key2f(best_key(spack[i])), l0, inv_t), tab)
                     : 0.0f;
        part += (double) w[t];
    }
    double incl = wave_scan_f64_dpp(part);
    if (norm) {
        const double sum = __shfl(incl, WAVE - 1, WAVE);
        part             = 0.0;
#pragma unroll
        for (int t = 0; t < IPT; ++t) {
            const int i = IPT * lane + t;
            w[t]        = i < n ? (float) ((double) w[t] / sum) : 0.0f;
            part += (double) w[t];
        }
        incl = wave_scan_f64_dpp(part);
    }
    double c[IPT]; /* inclusive prefix at each owned entry */
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

/* Workgroup-wide choice of one radix digit: hist[256] holds the counts of the current digit
 * among the keys that match the prefix; returns the digit that contains the `remaining`-th
 * largest key and updates `remaining` to the rank inside that digit. */
__device__ __forceinline__ int radix_pick_digit(const int *hist, int &remaining, int *s_scan,
                                                int *s_sel) {
    const int tid  = threadIdx.x;
    const int mine = hist[255 - tid]; /* thread t owns digit 255 - t: descending order */
    const int incl = block_scan_i32(mine, s_scan, nullptr);
    if (incl >= remaining && incl - mine < remaining) {
        s_sel[0] = 255 - tid;
        s_sel[1] = remaining - (incl - mine);
    }
    __syncthreads();
    const int digit = s_sel[0];
    remaining       = s_sel[1];
    __syncthreads();
    return digit;
}

/* LDS radix select: the k-th largest key of n packed entries held in LDS (1 <= k <= n). Returns
 * the key and how many of the entries equal to it are needed. */
__device__ uint32_t lds_kth_largest(const uint64_t *packs, int n, int k, int *hist, int *s_scan,
                                    int *s_sel, int &need_ties) {
    const int tid    = threadIdx.x;
    uint32_t  prefix = 0, mask = 0;
    int       remaining = k;
    for (int shift = 24; shift >= 0; shift -= 8) {
        hist[tid] = 0;
        __syncthreads();
        for (int i = tid; i < n; i += TPB) {
            const uint32_t key = best_key(packs[i]);
            if ((key & mask) == prefix)
                atomicAdd(&hist[(key >> shift) & 255u], 1);
        }
        __syncthreads();
        const int digit = radix_pick_digit(hist, remaining, s_scan, s_sel);
        prefix |= (uint32_t) digit << shift;
        mask |= 255u << shift;
    }
    need_ties = remaining;
    return prefix;
}

/* Bitonic sort of n (a power of two) packed entries in LDS, descending. */
__device__ void lds_sort_desc(uint64_t *s, int n) {
    for (int size = 2; size <= n; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            for (int t = threadIdx.x; t < n / 2; t += TPB) {
                const int      i    = 2 * t - (t & (stride - 1));
                const int      j    = i + stride;
                const bool     desc = (i & size) == 0;
                const uint64_t x = s[i], y = s[j];
                if ((x < y) == desc) {
                    s[i] = y;
                    s[j] = x;
                }
            }
            __syncthreads();
        }
    }
}

/* ============================================================================================
 * topk_row_general: exact top-k of one whole row by one workgroup, for any k up to the
 * capacity of `spack` and any data (masked rows full of -inf, all-equal rows, k in the
 * thousands). Four 8-bit radix passes over the row fix the k-th largest key (the LDS radix
 * select, no sort of the vocabulary); a fifth pass gathers everything above it plus, in index
 * order, as many of its ties as are still needed (sampler.c:207 orders equal logits by
 * ascending index). Leaves the k survivors sorted in spack[0..k) and returns k.
 * ========================================================================================== */
struct GeneralShared {
    int hist[256];
    int scan[NWAVES];
    int sel[2];
    int n;
};

template <int NV, bool PEN, bool MASK = true>
__device__ __forceinline__ int topk_row_general(const RowView &rv, int row, int k_want, uint64_t *spack,
                                int spack_cap, uint32_t *cnt16, GeneralShared &gs_) {
    constexpr int TILE = NV * TPB * 4;
    const int     tid  = threadIdx.x;
    const int     n    = rv.n_vocab;
    const int     k    = k_want < n ? k_want : n;
    float4        v[NV];

    uint32_t prefix = 0, mask = 0;
    int      remaining = k;
    for (int shift = 24; shift >= 0; shift -= 8) {
        gs_.hist[tid] = 0;
        __syncthreads();
        for (int base = 0; base < n; base += TILE) {
            const int end = base + TILE < n ? base + TILE : n;
            fetch_chunk<NV, PEN, MASK>(rv, row, rv.n_rows, base, end, cnt16, v);
#pragma unroll
            for (int j = 0; j < NV; ++j) {
                const int e = base + 4 * (j * TPB + tid);
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const uint32_t key = f2key(f4_get(v[j], c));
                    if (e + c < end && (key & mask) == prefix)
                        atomicAdd(&gs_.hist[(key >> shift) & 255u], 1);
                }
            }
            if (PEN)
                __syncthreads(); /* the count table is rebuilt by the next tile */
        }
        __syncthreads();
        const int digit = radix_pick_digit(gs_.hist, remaining, gs_.scan, gs_.sel);
        prefix |= (uint32_t) digit << shift;
        mask |= 255u << shift;
    }
    const uint32_t kth  = prefix;
    const int      need = remaining;

    if (tid == 0)
        gs_.n = 0;
    __syncthreads();
    int ties_before = 0;
    for (int base = 0; base < n; base += TILE) {
        const int end = base + TILE < n ? base + TILE : n;
        fetch_chunk<NV, PEN, MASK>(rv, row, rv.n_rows, base, end, cnt16, v);
        int ties_here = 0;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int e = base + 4 * (j * TPB + tid);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint32_t key = f2key(f4_get(v[j], c));
                if (e + c < end) {
                    if (key > kth) {
                        const int pos = atomicAdd(&gs_.n, 1);
                        if (pos < spack_cap)
                            spack[pos] = pack_best(key, (uint32_t) (e + c));
                    } else if (key == kth) {
                        ++ties_here;
                    }
                }
            }
        }
        if (__syncthreads_or(ties_here != 0 && ties_before < need)) {
            /* index order inside the tile is (j, thread, component) */
#pragma unroll
            for (int j = 0; j < NV; ++j) {
                const int e   = base + 4 * (j * TPB + tid);
                int       cnt = 0;
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    cnt += (e + c < end) && f2key(f4_get(v[j], c)) == kth;
                int       slab;
                const int incl = block_scan_i32(cnt, gs_.scan, &slab);
                int       ord  = ties_before + incl - cnt;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    if ((e + c < end) && f2key(f4_get(v[j], c)) == kth) {
                        if (ord < need) {
                            const int pos = atomicAdd(&gs_.n, 1);
                            if (pos < spack_cap)
                                spack[pos] = pack_best(kth, (uint32_t) (e + c));
                        }
                        ++ord;
                    }
                }
                ties_before += slab;
            }
        }
    }
    __syncthreads();
    /* pad to a power of two with entries that sort last, then order */
    int p2 = 1;
    while (p2 < k)
        p2 <<= 1;
    for (int i = k + tid; i < p2; i += TPB)
        spack[i] = 0;
    __syncthreads();
    lds_sort_desc(spack, p2);
    return k;
}

struct FinalArgs {
    int   mode; /* FINAL_ARGMAX, FINAL_TEMPERATURE, FINAL_TOPK */
    int   k;
    int   k_sel; /* rank of the thread maximum used as the bound (>= k) */
    float inv_t;
    float top_p;
    float min_p;
    const float   *uniforms;
    const uint64_t *chunk_best;
    const double   *chunk_sum;
    const double   *slab_sum; /* FINAL_TEMPERATURE: [rows][chunks][SLABS_MAX] */
    const float    *tmax;
    int32_t        *out;
    int32_t        *row_flag; /* FINAL_SORTED: 1 = the row goes on to the candidate list,
                               * 2 = to the whole-row walk */
    CandSpace       cand;
    double          ln_min_p; /* log(min_p), taken on the host */
    int             zb_min_p; /* last z bin that can hold an entry passing min_p (with slack);
                               * ZBINS - 1 when min_p is off or that deep */
    bool            minp_listed; /* the exp-sum pass listed every row up to that bin */
    bool            cap_after;   /* top-k: the scan ran on the logits before the soft-cap (the
                                  * thread maxima, the candidates); the row-final kernel applies
                                  * it to what it keeps. The cap tanhf(x / c) * c never turns the
                                  * order of two logits round (tanhf is monotone over every
                                  * binary32, tests/test_tanhf_exact.py), but it maps neighbouring
                                  * logits to the same value: only entries whose capped value lies
                                  * strictly above the capped bound are certain to be all there
                                  * is, and k of those are needed. */
};

/* ============================================================================================
 * topk_from_tmax: the row-final side of the thread-maxima path (see k_tmax_scan).
 *   1. each thread of this workgroup takes KPT of the row's thread maxima (entry q*256 + tid
 *      belongs to chunk q, scanning thread tid) and keeps their maximum;
 *   2. the k-th largest of 128 pairwise maxima of those bounds the k-th largest thread maximum,
 *      hence the row's k-th largest element, from below; every wavefront finds it on the
 *      leading 20 key bits by a bitwise search with ballots;
 *   3. the scanning threads at or above the bound are listed (about k ln-ish many);
 *   4. their 4*NV elements each are read again, penalised from the history counts of exactly
 *      those elements, soft-capped, and those reaching the bound are kept;
 *   5. the kept entries are ordered by counting and the first k are the row's top k, equal
 *      logits in ascending index order (sampler.c:207).
 * Returns true when the row has to take the general path instead (fewer than k real maxima,
 * long runs of equal values); otherwise k_out entries lie sorted in s_pack.
 * ========================================================================================== */
template <int NV, bool PEN, int KPT, bool MASK>
__device__ __forceinline__ bool topk_from_tmax(const RowView &rv, const FinalArgs &a, int row,
                                               uint8_t *slot, uint32_t *s_mx, int *s_selid,
                                               uint32_t *s_pcnt, uint64_t *s_m, uint64_t *s_pack,
                                               int *s_n, int *s_n2, int &k_out) {
    const int tid = threadIdx.x, lane = tid & (WAVE - 1);
    const int C   = rv.n_chunks;
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
    s_mx[tid] = f2key(mxf); /* 0 when the thread saw no real maximum */
    __syncthreads();
    /* 2 */
    const uint32_t a0 = s_mx[lane], a1 = s_mx[lane + 64], a2 = s_mx[lane + 128],
                   a3 = s_mx[lane + 192];
    int      real;
    uint32_t tau = 0u;
    if (a.k_sel <= 64) {
        /* 128 pairwise maxima: about -128 ln(1 - k/128) threads end up selected */
        const uint32_t m0 = a0 > a2 ? a0 : a2, m1 = a1 > a3 ? a1 : a3;
        real = __popcll(__ballot(m0 != 0u)) + __popcll(__ballot(m1 != 0u));
#pragma unroll
        for (int bit = 31; bit >= 12; --bit) {
            const uint32_t t   = tau | (1u << bit);
            const int      cnt = __popcll(__ballot(m0 >= t)) + __popcll(__ballot(m1 >= t));
            if (cnt >= a.k_sel)
                tau = t;
        }
    } else {
        /* all 256 maxima: about -256 ln(1 - k/256) threads */
        real = __popcll(__ballot(a0 != 0u)) + __popcll(__ballot(a1 != 0u)) +
               __popcll(__ballot(a2 != 0u)) + __popcll(__ballot(a3 != 0u));
#pragma unroll
        for (int bit = 31; bit >= 12; --bit) {
            const uint32_t t   = tau | (1u << bit);
            const int      cnt = __popcll(__ballot(a0 >= t)) + __popcll(__ballot(a1 >= t)) +
                            __popcll(__ballot(a2 >= t)) + __popcll(__ballot(a3 >= t));
            if (cnt >= a.k_sel)
                tau = t;
        }
    }
    /* keys at or below that of -inf: the bound says nothing (masked rows) */
    if (real < a.k_sel || tau < 0x00800000u)
        return true;
    const float bound = key2f(tau);
    /* what a kept element has to reach: the bound itself, or -- when the maxima were taken
     * before the soft-cap -- more than the capped bound (see FinalArgs::cap_after) */
    const float bound_kept = a.cap_after ? softcap1(bound, rv.softcap) : bound;
    /* 3 */
    uint32_t selmask = 0u;
#pragma unroll
    for (int q = 0; q < KPT; ++q)
        selmask |= (uint32_t) (raw[q] >= bound) << q;
    int pos = wave_reserve(__popc(selmask), s_n);
    while (selmask) { /* a few rounds: the selected maxima are spread over the threads */
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
        return true; /* long runs of equal maxima */
    /* 4 */
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
        const int shift = 31 - __clz(rv.per_chunk); /* per_chunk = 1024 * NV */
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
    /* survivors are appended in any order (the ranking below orders them): their keys wait in
     * registers until the lane has seen all its tasks, so that it asks for places once -- every
     * LDS atomic that returns a value costs the wavefront a round trip */
    uint32_t ck[TASKS][4];
    int      n_keep = 0;
#pragma unroll
    for (int q = 0; q < TASKS; ++q) {
        const int t = tid + q * TPB;
#pragma unroll
        for (int c = 0; c < 4; ++c)
            ck[q][c] = 0u;
        if (e0[q] >= e1[q])
            continue; /* no task (whole wavefronts beyond the list skip the block) */
        float x4[4] = {r[q].x, r[q].y, r[q].z, r[q].w};
        if (PEN) {
            const uint4 hc = *reinterpret_cast<const uint4 *>(&s_pcnt[t * 4]);
            if (hc.x | hc.y | hc.z | hc.w) { /* few float4 groups hold a history token */
                x4[0] = hc.x ? penalise(x4[0], hc.x, rv.rep, rv.inv_rep, rv.freq, rv.pres) : x4[0];
                x4[1] = hc.y ? penalise(x4[1], hc.y, rv.rep, rv.inv_rep, rv.freq, rv.pres) : x4[1];
                x4[2] = hc.z ? penalise(x4[2], hc.z, rv.rep, rv.inv_rep, rv.freq, rv.pres) : x4[2];
                x4[3] = hc.w ? penalise(x4[3], hc.w, rv.rep, rv.inv_rep, rv.freq, rv.pres) : x4[3];
            }
        }
        if (rv.softcap > 0.0f) {
#pragma unroll
            for (int c = 0; c < 4; ++c)
                x4[c] = softcap1(x4[c], rv.softcap);
        }
        const int      nvalid = e1[q] - e0[q]; /* 4 but at the row's end */
        const uint32_t ok     = (MASK && rv.allowed) ? allowed_nibble(rv, row, e0[q]) : 0xfu;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            /* (a NaN fails the comparison: keys are > 0) */
            if ((a.cap_after ? x4[c] > bound_kept : x4[c] >= bound_kept) && c < nvalid &&
                ((ok >> c) & 1u)) {
                ck[q][c] = f2key(x4[c]);
                ++n_keep;
            }
        }
    }
    if (n_keep) {
        int at = atomicAdd(s_n2, n_keep);
#pragma unroll
        for (int q = 0; q < TASKS; ++q) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if (ck[q][c]) {
                    if (at < TPB)
                        s_m[at] = pack_best(ck[q][c], (uint32_t) (e0[q] + c));
                    ++at;
                }
            }
        }
    }
    __syncthreads();
    const int m = *s_n2;
    /* m > 256: long runs of equal values at the bound. m < k can only happen when the thread
     * maxima were taken before the penalties (see the launch code): then too many of the
     * leading logits were penalised below the bound and it certifies nothing. */
    if (m > TPB || m < a.k)
        return true;
    const int k = a.k;
    /* 5: entry i is compared with the others by P = 256 / m2 <= 64 neighbouring lanes */
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
    if (i < m && part == 0 && rank < k)
        s_pack[rank] = me;
    __syncthreads();
    k_out = k;
    return false;
}

} // namespace gs
#include "sampler_walk.h"
#include "sampler_draw.h"
#include "sampler_sorted_prob.h"
#include "sampler_walk_coop.h"
#include "sampler_spec.h"
#include "sampler_draft.h"
#include "sampler_cands.h"
#include "sampler_cands_one_launch.h"
namespace gs {

/* ============================================================================================
 * Row-final kernels: one workgroup per row, one kernel per sampling mode.
 * ========================================================================================== */

/* argmax: sampler.c:52-62 */
__global__ __launch_bounds__(TPB) void k_final_argmax(RowView rv, FinalArgs a) {
    __shared__ uint64_t s_red[NWAVES];
    const int           row = blockIdx.x;
    const uint64_t      b   = row_best_from_chunks(a.chunk_best, row, rv.n_chunks, s_red);
    if (threadIdx.x == 0) {
        const float first = rv.logits[(long) row * rv.ld];
        /* a NaN at index 0 is never displaced by the strict '>' of the reference; after the
         * transforms it stays NaN, so the raw value decides (unless token 0 is forbidden) */
        const bool nan0 = first != first && (!rv.allowed || allowed_at(rv, row, 0));
        a.out[row]      = nan0 ? 0 : (int32_t) best_idx(b);
    }
}

/* temperature: sampler.c:90-102 over all n in index order: locate the chunk from the per-chunk
 * sums, then scan that chunk. */
template <int NV, bool PEN>
__global__ __launch_bounds__(TPB) void k_final_temperature(RowView rv, FinalArgs a) {
    __shared__ uint64_t   s_red[NWAVES];
    __shared__ uint64_t   s_tab[32];
    __shared__ WalkShared s_walk;
    __shared__ double     s_csum[MAX_CHUNKS];
    __shared__ __align__(16) uint32_t s_cnt16[PEN ? TPB * 2 : 1];
    const int row = blockIdx.x, tid = threadIdx.x, C = rv.n_chunks;
    if (tid < C)
        s_csum[tid] = a.chunk_sum[(long) row * C + tid];
    if (tid < 32)
        s_tab[tid] = g_expf_tab[tid];
    const float u_row = a.uniforms[row];
    const float mx    = key2f(best_key(row_best_from_chunks(a.chunk_best, row, C, s_red)));
    /* (row_best_from_chunks ends with a barrier: s_csum and the table are visible) */
    const int tok = index_order_walk<NV, PEN, false>(
        rv, row, (int) gridDim.x, s_csum, a.slab_sum + (long) row * C * SLABS_MAX, C, u_row, mx,
        a.inv_t, 0.0, nullptr, false, -1, s_tab, s_cnt16, s_walk);
    if (tid == 0)
        a.out[row] = tok;
}

/* top-p / min-p over the whole vocabulary (sampler.c:232-305): the thread-maxima shortcut; a
 * row it cannot serve raises its flag for the whole-row walk. */
template <int NV, bool PEN>
__global__ __launch_bounds__(TPB) void k_final_sorted(RowView rv, FinalArgs a) {
    __shared__ uint64_t s_red[NWAVES];
    __shared__ uint64_t s_tab[32];
    __shared__ __align__(16) uint8_t s_big[TMAX_LDS];
    __shared__ uint32_t s_mx[TPB];
    __shared__ int      s_selid[SEL_MAX];
    __shared__ __align__(16) uint32_t s_pcnt[PEN ? SEL_MAX * 4 * NV : 4];
    __shared__ uint64_t s_m[TPB];
    __shared__ uint64_t s_srt[TPB];
    __shared__ float    s_wt[TPB];
    __shared__ double   s_csum[MAX_CHUNKS];
    __shared__ int      s_n, s_n2;
    __shared__ double   s_sum;
    const int row = blockIdx.x, tid = threadIdx.x, C = rv.n_chunks;
    if (tid < 32)
        s_tab[tid] = g_expf_tab[tid];
    if (tid < C)
        s_csum[tid] = a.chunk_sum[(long) row * C + tid];
    const float u_row = a.uniforms[row];
    const float mx    = key2f(best_key(row_best_from_chunks(a.chunk_best, row, C, s_red)));
    if (tid == 0) {
        double tot = 0.0;
        for (int c = 0; c < C; ++c)
            tot += s_csum[c];
        s_sum = tot;
    }
    __syncthreads();
    const double sum = s_sum;
    int          tok = -1;
    if (sum != sum && !(a.min_p > 0.0f)) {
        /* A NaN, a +inf or nothing finite in the row: the sum is NaN, the reference neither takes
         * its argmax branch (sampler.c:243, `sum <= 0` is false) nor finds an end of the nucleus
         * or a slot for the draw among normalised probabilities that are all NaN, and answers
         * with the last entry of its sorted array (sampler.c:287-303) -- the last token, its
         * comparator calling all entries equal and the sort keeping their order. */
        if (tid == 0) {
            a.row_flag[row]  = 0;
            a.out[row]       = rv.n_vocab - 1;
            a.cand.path[row] = 1;
        }
        return;
    }
    if (a.minp_listed && a.cand.count[(long) row * CAND_COUNT_STRIDE] <= CAND_CAP) {
        /* the exp-sum pass listed the row under the min-p bound (holding softmax arguments, not pn): the list
         * walk serves it, top-p included -- the kept prefix is the shorter of the two */
        if (tid == 0) {
            const int   B      = a.zb_min_p;
            const float p_out  = geist_expf_glibc_le0(-(float) (B + 1) / (float) ZBIN_PER_NAT, s_tab);
            const float pn_out = (float) ((double) p_out / sum);
            a.cand.out_key[row]   = __float_as_uint(pn_out) + 1u;
            a.cand.row_bound[row] = B;
            a.cand.row_sum[row]   = sum;
            a.row_flag[row]       = 4;
            a.out[row]            = -1;
        }
        return;
    }
    if (C <= 16)
        tok = sorted_from_tmax<NV, PEN, 16>(rv, a, row, mx, sum, u_row, s_big, s_mx, s_wt, s_selid,
                                            s_pcnt, s_m, s_srt, &s_n, &s_n2, s_tab);
    else if (C <= TMAX_LDS / TPB)
        tok = sorted_from_tmax<NV, PEN, TMAX_LDS / TPB>(rv, a, row, mx, sum, u_row, s_big, s_mx,
                                                        s_wt, s_selid, s_pcnt, s_m, s_srt, &s_n,
                                                        &s_n2, s_tab);
    if (tok >= 0) {
        if (tid == 0) {
            a.row_flag[row]  = 0;
            a.out[row]       = tok;
            a.cand.path[row] = 1;
        }
        return;
    }
    /* The shortcut could not serve the row. Last z bin (z = (max - l) * inv_t) that can hold an
     * element of the kept prefix.
     *   top-p: estimated from ALL the row's thread maxima, binned by z with fast exponentials as
     *   weights. Where M of the T scanning threads have their maximum above a value, about
     *   -T ln(1 - M/T) elements lie above it if the vocabulary order is unrelated to the logits
     *   (each element beyond a thread's first hides behind that thread's maximum), so a bin's
     *   mass is scaled by 1 / (1 - M/T) at the bin. The first bin at which the scaled mass
     *   passes top_p plus a quarter of the rest, and one more bin, is taken. It is an estimate:
     *   the walk over the list sums the listed mass exactly and hands the row on to the
     *   whole-row walk when the kept prefix is not certainly inside the list.
     *   min-p: pn_i >= min_p * pn_0 needs z_i <= -ln(min_p), in closed form, taken with slack.
     *   Both set: the shorter prefix, so the smaller bin. */
    __syncthreads();
    constexpr int COPIES = 8; /* lanes spread over copies of the bins: fewer same-address adds */
    float        *s_zh   = reinterpret_cast<float *>(s_big);                      /* [COPIES][ZBINS] */
    int          *s_zc   = reinterpret_cast<int *>(s_big + COPIES * ZBINS * 4);   /* [COPIES][ZBINS] */
    static_assert(COPIES * ZBINS * 8 <= TMAX_LDS, "bins live in the slot table's space");
    const bool want_p = a.top_p > 0.0f && a.top_p < 1.0f;
    for (int i = tid; i < COPIES * ZBINS * 2; i += TPB)
        reinterpret_cast<uint32_t *>(s_big)[i] = 0u;
    __syncthreads();
    if (want_p) {
        const float *tm   = a.tmax + (long) row * C * TPB + tid;
        const int    copy = (tid & (COPIES - 1)) * ZBINS;
        const int    last = a.zb_min_p < ZBINS - 2 ? a.zb_min_p + 1 : ZBINS - 2; /* deeper bins cannot matter */
        for (int q = 0; q < C; ++q) {
            const float arg = softmax_arg(tm[(long) q * TPB], mx, a.inv_t);
            const int   zb  = zbin(arg); /* NaN (a thread without an element) lands past `last` */
            if (zb <= last) {
                atomicAdd(&s_zc[copy + zb], 1);
                unsafeAtomicAdd(&s_zh[copy + zb], __expf(arg));
            }
        }
    }
    __syncthreads();
    if (tid < WAVE) {
        int B = ZBINS - 1;
        if (want_p) {
            /* scanning threads that hold at least one element of the row */
            const int rem  = rv.n_vocab - (C - 1) * rv.per_chunk;
            const int T    = (C - 1) * TPB + ((rem + 3) / 4 < TPB ? (rem + 3) / 4 : TPB);
            const int b0   = 2 * tid, b1 = 2 * tid + 1;
            int       c0 = 0, c1 = 0;
            float     w0 = 0.f, w1 = 0.f;
#pragma unroll
            for (int k = 0; k < COPIES; ++k) {
                c0 += s_zc[k * ZBINS + b0];
                c1 += s_zc[k * ZBINS + b1];
                w0 += s_zh[k * ZBINS + b0];
                w1 += s_zh[k * ZBINS + b1];
            }
            const int    before = wave_scan_i32_dpp(c0 + c1) - c0 - c1;
            const double invT   = 1.0 / (double) (T > 0 ? T : 1);
            const double l0     = 1.0 - ((double) before + 0.5 * (double) c0) * invT;
            const double l1     = 1.0 - ((double) (before + c0) + 0.5 * (double) c1) * invT;
            const double s0     = (double) w0 / (l0 > 0.05 ? l0 : 0.05);
            const double s1     = (double) w1 / (l1 > 0.05 ? l1 : 0.05);
            const double incl   = wave_scan_f64_dpp(s0 + s1);
            const double need   = ((double) a.top_p + 0.25 * (1.0 - (double) a.top_p)) * sum;
            const uint64_t h0   = __ballot(incl - s1 >= need && b0 < ZBINS - 1);
            const uint64_t h1   = __ballot(incl >= need && b1 < ZBINS - 1);
            int            first = ZBINS;
            if (h0)
                first = 2 * (__ffsll((long long) h0) - 1);
            if (h1) {
                const int f1 = 2 * (__ffsll((long long) h1) - 1) + 1;
                first        = f1 < first ? f1 : first;
            }
            if (first < ZBINS - 1)
                B = first + 1 < ZBINS - 1 ? first + 1 : first; /* one more bin for the estimate */
        }
        B = a.zb_min_p < B ? a.zb_min_p : B;
        if (tid == 0) {
            /* an element outside the list has z >= (B + 1) / ZBIN_PER_NAT (the product in zbin()
             * is exact), so its p is at most expf of minus that; one step up covers any
             * non-monotonic last bit of expf or of the division */
            const float p_out  = geist_expf_glibc_le0(-(float) (B + 1) / (float) ZBIN_PER_NAT, s_tab);
            const float pn_out = (float) ((double) p_out / sum);
            a.cand.out_key[row]   = __float_as_uint(pn_out) + 1u;
            a.cand.row_bound[row] = B;
            a.cand.count[(long) row * CAND_COUNT_STRIDE]     = 0;
            a.row_flag[row]       = B < ZBINS - 1 ? 1 : 2;
            a.out[row]            = -1;
        }
    }
}

/* top-k (sampler.c:178-228) and the chain behind it: select from the row's thread maxima, then
 * gather; rows the shortcut cannot serve (masked rows full of -inf, all-equal rows, tiny or huge
 * vocabularies) select over the whole row in place. */
template <int NV, bool PEN, bool MASK>
__global__ __launch_bounds__(TPB) void k_final_topk(RowView rv, FinalArgs a) {
    __shared__ uint64_t      s_tab[32];
    __shared__ GeneralShared s_gs;
    __shared__ __align__(16) uint8_t s_big[TMAX_LDS];
    __shared__ uint32_t      s_mx[TPB];
    __shared__ int           s_selid[SEL_MAX];
    __shared__ __align__(16) uint32_t s_pcnt[PEN ? SEL_MAX * 4 * NV : 4];
    __shared__ uint64_t      s_m[TPB];
    __shared__ uint64_t      s_pack[TOPK_FAST_MAX];
    __shared__ __align__(16) uint32_t s_cnt16[PEN ? NV * TPB * 2 : 1];
    __shared__ int           s_n, s_n2;
    const int row = blockIdx.x, tid = threadIdx.x, C = rv.n_chunks;
    if (tid < 32)
        s_tab[tid] = g_expf_tab[tid];
    const float u_row   = a.uniforms[row];
    int         k       = 0;
    bool        general = true;
    if (C <= 16)
        general = topk_from_tmax<NV, PEN, 16, MASK>(rv, a, row, s_big, s_mx, s_selid, s_pcnt, s_m,
                                              s_pack, &s_n, &s_n2, k);
    else if (C <= TMAX_LDS / TPB)
        general = topk_from_tmax<NV, PEN, TMAX_LDS / TPB, MASK>(rv, a, row, s_big, s_mx, s_selid,
                                                                s_pcnt,
                                                          s_m, s_pack, &s_n, &s_n2, k);
    if (general) {
        __syncthreads();
        k = topk_row_general<NV, PEN, MASK>(rv, row, a.k, s_pack, TOPK_FAST_MAX, s_cnt16, s_gs);
    }
    /* k <= TOPK_FAST_MAX = 128: the tail runs on one wavefront without barriers */
    if (tid < WAVE) {
        const int tok =
            k <= WAVE ? finish_sorted_wave<1>(k, s_pack, a.inv_t, a.top_p, a.min_p, u_row, s_tab)
                      : finish_sorted_wave<2>(k, s_pack, a.inv_t, a.top_p, a.min_p, u_row, s_tab);
        if (tid == 0)
            a.out[row] = tok;
    }
}

/* ============================================================================================
 * k_topk_general: top-k for k above the candidate path's limit (up to 8192, the reference's own
 * cap, sampler.c:213-215). One workgroup per row; the survivors live in dynamic LDS.
 * ========================================================================================== */
template <int NV, bool PEN>
__global__ __launch_bounds__(TPB) void k_topk_general(RowView rv, FinalArgs a, int spack_cap) {
    extern __shared__ uint64_t s_dyn_pack[];
    __shared__ FinishShared    s_fs;
    __shared__ GeneralShared   s_gs;
    __shared__ __align__(16) uint32_t s_cnt16[PEN ? NV * TPB * 2 : 1];
    const int                  row = blockIdx.x;
    const int k = topk_row_general<NV, PEN>(rv, row, a.k, s_dyn_pack, spack_cap, s_cnt16, s_gs);
    const int tok =
        finish_sorted(k, s_dyn_pack, a.inv_t, a.top_p, a.min_p, a.uniforms[row], s_fs);
    if (threadIdx.x == 0)
        a.out[row] = tok;
}

/* ============================================================================================
 * k_write_probs: pn_i = (float)((double)p_i / sum), sampler.c:246-253.
 * ========================================================================================== */
template <int NV, bool PEN>
__global__ __launch_bounds__(TPB) void k_write_probs(RowView rv, float inv_t,
                                                     const uint64_t *__restrict__ chunk_best,
                                                     const double *__restrict__ chunk_sum,
                                                     float *__restrict__ probs, long ld_probs,
                                                     const int32_t *__restrict__ row_flag) {
    __shared__ __align__(16) uint32_t s_cnt16[PEN ? NV * TPB * 2 : 1];
    __shared__ uint64_t s_red[NWAVES];
    __shared__ uint64_t s_tab[32];
    __shared__ double   s_total;
    const int           row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
    if (row_flag && row_flag[row] != 2)
        return; /* only the rows that asked for their probabilities */
    if (tid < 32)
        s_tab[tid] = g_expf_tab[tid];
    if (tid == 0) {
        double t = 0.0;
        for (int c = 0; c < rv.n_chunks; ++c)
            t += chunk_sum[(long) row * rv.n_chunks + c];
        s_total = t;
    }
    int base, end;
    chunk_bounds<NV>(rv, chunk, base, end);
    float4 v[NV];
    fetch_chunk<NV, PEN>(rv, row, (int) gridDim.y, base, end, s_cnt16, v);
    const float  mx  = key2f(best_key(row_best_from_chunks(chunk_best, row, rv.n_chunks, s_red)));
    const double tot = s_total;
    float       *out = probs + (long) row * ld_probs;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int e = base + 4 * (j * TPB + tid);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            if (e + c < end) {
                const float p = geist_expf_glibc_le0(softmax_arg(f4_get(v[j], c), mx, inv_t), s_tab);
                out[e + c]    = (float) ((double) p / tot);
            }
        }
    }
}

/* ============================================================================================
 * Log-probability scoring: log_softmax(row)[token] for K tokens per row, as the reference's
 * evaluation tool computes it from peeked logits (tools/eval_geist.c:63-73 over
 * geist_session_peek_logits, src/archs/transformer/arch.c:167-197, which hands out the soft-capped
 * values): fp32 max, double exp of the fp32 difference, double sum, then
 * (double)(l[token] - max) - log(sum). Only K doubles per row leave the device.
 *   k_chunk_lse      grid (chunks, rows): sum of exp((double)(l - max)) over the chunk
 *   k_final_logprob  grid (rows): log of the row's sum, then the K values
 * ========================================================================================== */
template <int NV>
__global__ __launch_bounds__(TPB) void k_chunk_lse(RowView rv, const uint64_t *__restrict__ chunk_best,
                                                   double *__restrict__ chunk_sum) {
    __shared__ uint64_t s_red[NWAVES];
    __shared__ double   s_sum[NWAVES];
    int                 row, chunk;
    xcd_row_chunk(row, chunk);
    const int tid = threadIdx.x;
    int       base, end;
    chunk_bounds<NV>(rv, chunk, base, end);
    float4 v[NV];
    fetch_chunk<NV, false>(rv, row, (int) gridDim.y, base, end, nullptr, v);
    const float mx  = key2f(best_key(row_best_from_chunks(chunk_best, row, rv.n_chunks, s_red)));
    double      acc = 0.0;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int e = base + 4 * (j * TPB + tid);
#pragma unroll
        for (int c = 0; c < 4; ++c)
            if (e + c < end)
                acc += exp((double) __fsub_rn(f4_get(v[j], c), mx));
    }
    acc = block_sum_f64(acc, s_sum);
    if (tid == 0)
        chunk_sum[(long) row * rv.n_chunks + chunk] = acc;
}

__global__ __launch_bounds__(TPB) void k_final_logprob(RowView rv,
                                                       const uint64_t *__restrict__ chunk_best,
                                                       const double *__restrict__ chunk_sum,
                                                       const int32_t *__restrict__ tokens,
                                                       long tokens_ld, int k_per_row,
                                                       double *__restrict__ out, long out_ld) {
    __shared__ uint64_t s_red[NWAVES];
    __shared__ double   s_lse;
    const int           row = blockIdx.x, tid = threadIdx.x, C = rv.n_chunks;
    const float mx = key2f(best_key(row_best_from_chunks(chunk_best, row, C, s_red)));
    if (tid == 0) {
        double tot = 0.0;
        for (int c = 0; c < C; ++c)
            tot += chunk_sum[(long) row * C + c];
        s_lse = log(tot);
    }
    __syncthreads();
    const double lse = s_lse;
    for (int j = tid; j < k_per_row; j += TPB) {
        const int t = tokens[(long) row * tokens_ld + j];
        double    r = __builtin_nan("");
        if (t >= 0 && t < rv.n_vocab) {
            float x = rv.logits[(long) row * rv.ld + t];
            if (rv.softcap > 0.0f)
                x = softcap1(x, rv.softcap);
            r = (double) __fsub_rn(x, mx) - lse;
        }
        out[(long) row * out_ld + j] = r;
    }
}

/* ============================================================================================
 * k_penalties: in-place penalties; only the penalised positions are written back.
 * ========================================================================================== */
template <int NV>
__global__ __launch_bounds__(TPB) void k_penalties(RowView rv, float *__restrict__ logits_rw) {
    __shared__ __align__(16) uint32_t s_cnt16[NV * TPB * 2];
    const int           row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
    int                 base, end;
    chunk_bounds<NV>(rv, chunk, base, end);
    const HistPrefetch pf = history_prefetch(rv, row, (int) gridDim.y);
    history_clear<NV * TPB * 4>(s_cnt16);
    history_count(rv, row, pf, base, end, s_cnt16);
    float *rowp = logits_rw + (long) row * rv.ld;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int      off = 4 * (j * TPB + tid);
        const uint32_t w0 = s_cnt16[(off >> 1) + 0], w1 = s_cnt16[(off >> 1) + 1];
        if (w0 | w1) {
            const uint32_t cnt[4] = {w0 & 0xffffu, w0 >> 16, w1 & 0xffffu, w1 >> 16};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int e = base + off + c;
                if (cnt[c] && e < end)
                    rowp[e] = penalise(rowp[e], cnt[c], rv.rep, rv.inv_rep, rv.freq, rv.pres);
            }
        }
    }
}

/* ============================================================================================
 * k_rng_units: xorshift64* (sampler.c:35-48). shared: one state, row r takes draw r+1.
 * ========================================================================================== */
__device__ __forceinline__ uint64_t xorshift_step(uint64_t &s) {
    s ^= s >> 12;
    s ^= s << 25;
    s ^= s >> 27;
    return s * 0x2545F4914F6CDD1DULL;
}
__global__ void k_rng_units(uint64_t *states, int shared, int rows, float *uniforms) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (shared) {
        if (r == 0) {
            uint64_t s = states[0];
            for (int i = 0; i < rows; ++i)
                uniforms[i] = (float) (uint32_t) (xorshift_step(s) >> 40) * (1.0f / 16777216.0f);
            states[0] = s;
        }
        return;
    }
    if (r < rows) {
        uint64_t s  = states[r];
        uniforms[r] = (float) (uint32_t) (xorshift_step(s) >> 40) * (1.0f / 16777216.0f);
        states[r]   = s;
    }
}

} // namespace gs

/* ============================================================================================
 * Host-side launchers (plain functions; the C ABI in sampler_abi.hip validates shapes first).
 * ========================================================================================== */
namespace gs {

template <typename F>
static void dispatch(int nv, bool pen, F &&f) {
    if (nv == 8) {
        if (pen)
            f(std::integral_constant<int, 8>{}, std::true_type{});
        else
            f(std::integral_constant<int, 8>{}, std::false_type{});
    } else {
        if (pen)
            f(std::integral_constant<int, 2>{}, std::true_type{});
        else
            f(std::integral_constant<int, 2>{}, std::false_type{});
    }
}
#define GS_NV decltype(nv)::value
#define GS_PEN decltype(pen)::value

int launch_scan_expsum(const Launch &L, float inv_t, float *tmax, uint64_t *chunk_best,
                        double *chunk_sum, const int32_t *probe_token, int probe_L, float *probe_p,
                        const CandSpace *list, int zb_list, double *slab_sum, const MeetSpace &meet,
                        bool fast) {
    const dim3 grid(L.rv.n_chunks, L.rows), block(TPB);
    auto go = [&](auto kernel) {
        kernel<<<grid, block, 0, L.stream>>>(L.rv, inv_t, tmax, chunk_best, chunk_sum,
                                             list ? nullptr : slab_sum, probe_token, probe_L, probe_p,
                                             list ? *list : CandSpace{}, list ? zb_list : 0, meet);
    };
    if (fast && !list && !L.pen) { /* the tolerance mode's form without a meeting */
        if (L.nv == 8)
            slab_sum ? go(k_scan_expsum<8, false, false, true, true, true>)
                     : go(k_scan_expsum<8, false, false, false, true, true>);
        else
            slab_sum ? go(k_scan_expsum<2, false, false, true, true, true>)
                     : go(k_scan_expsum<2, false, false, false, true, true>);
        if (slab_sum)
            k_rescale_sums<true><<<dim3(L.rows), dim3(WAVE), 0, L.stream>>>(
                L.rv, inv_t, chunk_best, chunk_sum, slab_sum, probe_token, probe_L, probe_p);
        else
            k_rescale_sums<false><<<dim3(L.rows), dim3(WAVE), 0, L.stream>>>(
                L.rv, inv_t, chunk_best, chunk_sum, nullptr, probe_token, probe_L, probe_p);
        return 0;
    }
    if (list && L.nv == 8) {
        if (L.pen)
            fast ? go(k_scan_expsum<8, true, true, false, true>) : go(k_scan_expsum<8, true, true, false>);
        else
            fast ? go(k_scan_expsum<8, false, true, false, true>) : go(k_scan_expsum<8, false, true, false>);
        return 0;
    }
    dispatch(L.nv, L.pen, [&](auto nv, auto pen) {
        if (slab_sum)
            fast ? go(k_scan_expsum<GS_NV, GS_PEN, false, true, true>)
                 : go(k_scan_expsum<GS_NV, GS_PEN, false, true>);
        else
            fast ? go(k_scan_expsum<GS_NV, GS_PEN, false, false, true>)
                 : go(k_scan_expsum<GS_NV, GS_PEN, false, false>);
    });
    return 0;
}

int zbin_of_min_p(float min_p) {
    if (!(min_p > 0.0f))
        return ZBINS - 1;
    /* pn_i >= min_p * pn_0 needs z_i <= -ln(min_p); slack for the fp32 steps in between */
    const double z_m = -std::log((double) min_p) + 2e-3;
    return z_m * ZBIN_PER_NAT < (double) (ZBINS - 1) ? (int) (z_m * ZBIN_PER_NAT) : ZBINS - 1;
}

void launch_temperature_draw(const Launch &L, float inv_t, const float *uniforms, int32_t *out,
                             const MeetSpace &meet) {
    /* for launches of a few rows: the geometry of 2048 elements per workgroup only. Rows in
     * eights, so that the workgroups of a row have linear ids equal modulo 8 and share an XCD
     * (xcd_row_chunk); the workgroups of the rows that are not there leave at once. */
    const dim3 grid(L.rv.n_chunks, (L.rows + 7) & ~7), block(TPB);
    if (L.pen)
        k_temperature_draw<2, true><<<grid, block, 0, L.stream>>>(L.rv, L.rows, inv_t, uniforms, out, meet);
    else
        k_temperature_draw<2, false><<<grid, block, 0, L.stream>>>(L.rv, L.rows, inv_t, uniforms, out, meet);
}

void launch_spec(const Launch &L, const SpecLaunch &sp, const MeetSpace *meet) {
    SpecArgs a;
    a.L          = sp.L;
    a.greedy     = sp.greedy;
    a.inv_t      = sp.inv_t;
    a.q          = sp.q;
    a.ld_q       = sp.ld_q;
    a.draft      = sp.draft;
    a.uniforms   = sp.uniforms;
    a.chunk_best = sp.chunk_best;
    a.chunk_sum  = sp.chunk_sum;
    a.probe_p    = sp.probe_p;
    a.resid_sum  = sp.resid_sum;
    a.resid_slab = sp.resid_slab;
    a.slab_sum   = sp.slab_sum;
    a.out_tokens = sp.out_tokens;
    a.n_accepted = sp.n_accepted;
    const dim3   block(TPB);
    SpecVerdict *vd = static_cast<SpecVerdict *>(sp.verdict);
    if (sp.greedy) {
        k_spec_accept<<<dim3(sp.n_seq), block, 0, L.stream>>>(L.rv, a, vd);
    } else if (meet) { /* the residual and the draw in one launch */
        const dim3 grid(L.rv.n_chunks, sp.n_seq);
        if (L.nv == 8)
            k_spec_resid_draw<8><<<grid, block, 0, L.stream>>>(L.rv, a, vd, *meet);
        else
            k_spec_resid_draw<2><<<grid, block, 0, L.stream>>>(L.rv, a, vd, *meet);
        return;
    } else {
        const dim3 grid(L.rv.n_chunks, sp.n_seq);
        if (L.nv == 8)
            k_spec_resid<8><<<grid, block, 0, L.stream>>>(L.rv, a, vd);
        else
            k_spec_resid<2><<<grid, block, 0, L.stream>>>(L.rv, a, vd);
    }
    if (L.nv == 8)
        k_spec_final<8><<<dim3(sp.n_seq), block, 0, L.stream>>>(L.rv, a, vd);
    else
        k_spec_final<2><<<dim3(sp.n_seq), block, 0, L.stream>>>(L.rv, a, vd);
}

void launch_tmax_scan(const Launch &L, float *tmax, uint64_t *chunk_best, int32_t *zero_per_row) {
    const dim3 grid(L.rv.n_chunks, L.rows), block(TPB);
    dispatch(L.nv, L.pen, [&](auto nv, auto pen) {
        if (chunk_best)
            k_tmax_scan<GS_NV, GS_PEN, true><<<grid, block, 0, L.stream>>>(L.rv, tmax, chunk_best,
                                                                          zero_per_row);
        else
            k_tmax_scan<GS_NV, GS_PEN, false><<<grid, block, 0, L.stream>>>(L.rv, tmax, nullptr,
                                                                           nullptr);
    });
}

static FinalArgs final_args(const FinalLaunch &f) {
    FinalArgs a;
    a.mode       = f.mode;
    a.k          = f.k;
    a.k_sel      = f.k_sel > f.k ? f.k_sel : f.k;
    a.inv_t      = f.inv_t;
    a.top_p      = f.top_p;
    a.min_p      = f.min_p;
    a.uniforms   = f.uniforms;
    a.chunk_best = f.chunk_best;
    a.chunk_sum  = f.chunk_sum;
    a.slab_sum   = f.slab_sum;
    a.tmax       = f.tmax;
    a.row_flag   = f.row_flag;
    a.out        = f.out;
    a.cand       = f.cand;
    a.ln_min_p   = f.min_p > 0.0f ? std::log((double) f.min_p) : 0.0;
    a.zb_min_p    = zbin_of_min_p(f.min_p);
    a.minp_listed = f.minp_listed;
    a.cap_after   = f.cap_after;
    return a;
}

int cand_lanes_for(int k_eff, size_t n_vocab) {
    const double lam = 2048.0 * (double) k_eff / (double) n_vocab;
    double       p = std::exp(-lam), cdf = p; /* P(X <= m) for X ~ Poisson(lam) */
    int          m = 0;
    while (1.0 - cdf > 1e-8 && m < 64) {
        ++m;
        p *= lam / m;
        cdf += p;
    }
    ++m; /* P(X >= m) <= 1e-8 */
    if (m < 4)
        m = 4;
    return m <= CAND_LANES_MAX ? m : 0;
}

void launch_cand_scan(const Launch &L, float *tmax, const WaveCands &wc, int m) {
    const dim3 grid(L.rv.n_chunks, L.rows), block(TPB);
    k_cand_scan<8><<<grid, block, 0, L.stream>>>(L.rv, tmax, wc, m);
}

void launch_final_cand(const Launch &L, const FinalLaunch &f, const WaveCands &wc) {
    const FinalArgs a = final_args(f);
    const dim3      grid(L.rows), block(FC_THREADS);
    if (L.rv.n_chunks <= 16) { /* up to 64 scanning wavefronts per row */
        if (L.pen)
            k_final_cand<8, true, false><<<grid, block, 0, L.stream>>>(L.rv, a, wc);
        else
            k_final_cand<8, false, false><<<grid, block, 0, L.stream>>>(L.rv, a, wc);
    } else {
        if (L.pen)
            k_final_cand<8, true, true><<<grid, block, 0, L.stream>>>(L.rv, a, wc);
        else
            k_final_cand<8, false, true><<<grid, block, 0, L.stream>>>(L.rv, a, wc);
    }
}

#ifndef GS_RANK_TAIL
#define GS_RANK_TAIL 1e-8
#endif
int cand_rank_for(int k_eff, size_t n_vocab, size_t elems) {
    if (k_eff < 1 || elems == 0 || elems > n_vocab)
        return 0;
    int r = k_eff; /* the workgroup holds the whole row */
    if (elems < n_vocab) {
        /* P(X >= r) <= 1e-8 for X ~ Binomial(k_eff, share) */
        const double share = (double) elems / (double) n_vocab;
        double       p = std::pow(1.0 - share, k_eff), cdf = p;
        int          x = 0;
        while (1.0 - cdf > GS_RANK_TAIL && x < k_eff) {
            p *= (double) (k_eff - x) / (double) (x + 1) * share / (1.0 - share);
            ++x;
            cdf += p;
        }
        r = x + 1 < k_eff ? x + 1 : k_eff;
    }
    return r <= OL_RANK_MAX ? r : 0;
}

void launch_cand_scan_final(const Launch &scan, const Launch &L, const FinalLaunch &f, float *tmax,
                            const WgCands &wc, int r_w, int r_last, uint32_t *arrive,
                            bool far_always, const Notify &nt, int wgs_per_row, int groups) {
    const FinalArgs a = final_args(f);
    /* rows in eights: the workgroups of a row then have linear ids equal modulo 8 and share an
     * XCD; the workgroups of the rows that are not there leave at once */
    const dim3      grid(wgs_per_row, (L.rows + 7) & ~7), block(OL_THREADS);
    auto go = [&](auto kernel) {
        kernel<<<grid, block, 0, L.stream>>>(scan.rv, L.rv, wc, r_w, r_last, a, tmax, arrive,
                                             far_always ? 1 : 0, nt);
    };
    if (groups == 4) { /* launches of few rows: half the logits to a workgroup */
        if (L.pen)
            scan.rv.stream_loads ? go(k_cand_scan_final<true, true, 4>) : go(k_cand_scan_final<true, false, 4>);
        else
            scan.rv.stream_loads ? go(k_cand_scan_final<false, true, 4>) : go(k_cand_scan_final<false, false, 4>);
        return;
    }
    if (L.pen)
        scan.rv.stream_loads ? go(k_cand_scan_final<true, true, 8>) : go(k_cand_scan_final<true, false, 8>);
    else
        scan.rv.stream_loads ? go(k_cand_scan_final<false, true, 8>) : go(k_cand_scan_final<false, false, 8>);
}

__global__ __launch_bounds__(TPB) void k_zero_words(uint64_t *__restrict__ p, uint32_t n) {
    for (uint32_t i = blockIdx.x * TPB + threadIdx.x; i < n; i += gridDim.x * TPB)
        p[i] = 0ull;
}

void launch_zero_words(hipStream_t stream, uint64_t *p, uint32_t n) {
    if (n == 0)
        return;
    const uint32_t blocks = (n + TPB - 1) / TPB;
    k_zero_words<<<dim3(blocks < 64u ? blocks : 64u), dim3(TPB), 0, stream>>>(p, n);
}

__global__ void k_publish_epoch(Notify nt) {
    /* (the kernels before this one on the stream have ended: their stores are where the host
     * reads them) */
    __hip_atomic_store(nt.h_done, nt.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

void launch_publish_epoch(hipStream_t stream, const Notify &nt) {
    if (nt.h_done)
        k_publish_epoch<<<dim3(1), dim3(1), 0, stream>>>(nt);
}

int probe_workgroup_placement(hipStream_t stream, bool *same_xcd) {
    /* a grid shaped like the fused kernel's: do workgroups whose linear ids are equal modulo 8
     * run on one XCD? */
    const int gx = 4, gy = 64, n = gx * gy;
    int32_t  *d  = nullptr;
    int32_t   h[gx * gy];
    *same_xcd    = false;
    hipError_t e = hipMalloc((void **) &d, n * sizeof(int32_t));
    if (e != hipSuccess)
        return (int) e;
    k_xcd_of_workgroups<<<dim3(gx, gy), dim3(OL_THREADS), 0, stream>>>(d);
    e = hipMemcpyAsync(h, d, n * sizeof(int32_t), hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess)
        e = hipStreamSynchronize(stream);
    (void) hipFree(d);
    if (e != hipSuccess)
        return (int) e;
    bool ok = true;
    for (int i = 8; i < n; ++i)
        ok = ok && h[i] == h[i & 7];
    *same_xcd = ok;
    return 0;
}

void launch_row_final(const Launch &L, const FinalLaunch &f) {
    const FinalArgs a = final_args(f);
    const dim3 grid(L.rows), block(TPB);
    if (f.mode == FINAL_ARGMAX) {
        k_final_argmax<<<grid, block, 0, L.stream>>>(L.rv, a);
        return;
    }
    dispatch(L.nv, L.pen, [&](auto nv, auto pen) {
        if (f.mode == FINAL_TEMPERATURE)
            k_final_temperature<GS_NV, GS_PEN><<<grid, block, 0, L.stream>>>(L.rv, a);
        else if (f.mode == FINAL_SORTED)
            k_final_sorted<GS_NV, GS_PEN><<<grid, block, 0, L.stream>>>(L.rv, a);
        else if (L.rv.allowed)
            k_final_topk<GS_NV, GS_PEN, true><<<grid, block, 0, L.stream>>>(L.rv, a);
        else
            k_final_topk<GS_NV, GS_PEN, false><<<grid, block, 0, L.stream>>>(L.rv, a);
    });
}

int launch_topk_general(const Launch &L, const FinalLaunch &f) {
    FinalArgs a{};
    a.mode     = FINAL_TOPK;
    a.k        = f.k;
    a.inv_t    = f.inv_t;
    a.top_p    = f.top_p;
    a.min_p    = f.min_p;
    a.uniforms = f.uniforms;
    a.out      = f.out;
    int p2     = 1;
    while (p2 < f.k)
        p2 <<= 1;
    const size_t dyn = (size_t) p2 * sizeof(uint64_t);
    const dim3   grid(L.rows), block(TPB);
    hipError_t   e = hipSuccess;
    if (L.pen) {
        e = hipFuncSetAttribute((const void *) k_topk_general<4, true>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int) dyn);
        if (e == hipSuccess)
            k_topk_general<4, true><<<grid, block, dyn, L.stream>>>(L.rv, a, p2);
    } else {
        e = hipFuncSetAttribute((const void *) k_topk_general<4, false>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int) dyn);
        if (e == hipSuccess)
            k_topk_general<4, false><<<grid, block, dyn, L.stream>>>(L.rv, a, p2);
    }
    return (int) e;
}

void launch_write_probs(const Launch &L, float inv_t, const uint64_t *chunk_best,
                        const double *chunk_sum, float *probs, long ld_probs,
                        const int32_t *row_flag) {
    const dim3 grid(L.rv.n_chunks, L.rows), block(TPB);
    dispatch(L.nv, L.pen, [&](auto nv, auto pen) {
        k_write_probs<GS_NV, GS_PEN><<<grid, block, 0, L.stream>>>(
            L.rv, inv_t, chunk_best, chunk_sum, probs, ld_probs, row_flag);
    });
}

int configure_device_kernels() {
    /* k_sorted_candidates keeps a whole candidate list in LDS: more than the static limit */
    const int   dyn = CAND_CAP * (int) sizeof(uint32_t);
    const void *kernels[] = {(const void *) k_sorted_candidates<2, false>,
                             (const void *) k_sorted_candidates<2, true>,
                             (const void *) k_sorted_candidates<8, false>,
                             (const void *) k_sorted_candidates<8, true>};
    for (const void *k : kernels) {
        const hipError_t e =
            hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, dyn);
        if (e != hipSuccess)
            return (int) e;
    }
    return 0;
}

size_t walk_coop_bytes(size_t rows) { return rows * sizeof(CoopRow); }

void launch_candidates(const Launch &L, const FinalLaunch &f, float *probs, long ld_probs,
                       const WalkCoop &wc) {
    const dim3 grid(L.rv.n_chunks, L.rows), block(TPB);
    const int  dyn = CAND_CAP * (int) sizeof(uint32_t); /* see configure_device_kernels() */
    SortedRowArgs g;
    g.inv_t      = f.inv_t;
    g.chunk_best = f.chunk_best;
    g.chunk_sum  = f.chunk_sum;
    g.probs      = probs;
    g.ld_probs   = ld_probs;
    /* the cooperative whole-row walk holds a chunk of 8192 in registers */
    const int defer = wc.rows != nullptr && wc.spread && L.nv == 8 ? 1 : 0;
    if (f.minp_direct) {
        /* the exp-sum pass has listed every row: no row-final kernel, no listing pass. An
         * unlisted element lies in z bin zb + 1 or beyond; the same expf as on the device. */
        static const uint64_t tab[32] = GEIST_EXPF_TABLE_INIT;
        const int             zb      = zbin_of_min_p(f.min_p);
        const float p_out = geist_expf_glibc_le0(-(float) (zb + 1) / (float) ZBIN_PER_NAT, tab);
        dispatch(L.nv, L.pen, [&](auto nv, auto pen) {
            k_sorted_candidates<GS_NV, GS_PEN><<<dim3(L.rows), block, dyn, L.stream>>>(
                L.rv, g, f.cand, f.top_p, f.min_p, f.uniforms, f.row_flag, f.out, f.chunk_sum,
                L.rv.n_chunks, p_out, defer, wc.hint, wc.call);
        });
    } else {
        dispatch(L.nv, L.pen, [&](auto nv, auto pen) {
            k_list_candidates<GS_NV, GS_PEN><<<grid, block, 0, L.stream>>>(
                L.rv, f.inv_t, f.chunk_best, f.chunk_sum, f.row_flag, f.cand);
            k_sorted_candidates<GS_NV, GS_PEN><<<dim3(L.rows), block, dyn, L.stream>>>(
                L.rv, g, f.cand, f.top_p, f.min_p, f.uniforms, f.row_flag, f.out, nullptr, 0, 0.0f,
                defer, wc.hint, wc.call);
        });
    }
    if (defer) {
        /* the rows flagged 2, a workgroup per chunk */
        if (wc.clear)
            launch_zero_words(L.stream, static_cast<uint64_t *>(wc.rows),
                              (uint32_t) (walk_coop_bytes((size_t) L.rows) / sizeof(uint64_t)));
        CoopRow *cr = static_cast<CoopRow *>(wc.rows);
        if (L.pen)
            k_whole_row_coop<8, true><<<grid, block, 0, L.stream>>>(
                L.rv, g, f.cand, f.top_p, f.min_p, f.uniforms, f.row_flag, f.out, cr, wc.step_base,
                wc.wait_limit, wc.hint, wc.call);
        else
            k_whole_row_coop<8, false><<<grid, block, 0, L.stream>>>(
                L.rv, g, f.cand, f.top_p, f.min_p, f.uniforms, f.row_flag, f.out, cr, wc.step_base,
                wc.wait_limit, wc.hint, wc.call);
        /* rows that are still flagged 2 (a wait ran out, sums that are not finite): one workgroup
         * each, as without the spread walk */
        dispatch(L.nv, L.pen, [&](auto nv, auto pen) {
            k_sorted_candidates<GS_NV, GS_PEN><<<dim3(L.rows), block, dyn, L.stream>>>(
                L.rv, g, f.cand, f.top_p, f.min_p, f.uniforms, f.row_flag, f.out, nullptr, 0, 0.0f,
                0, nullptr, 0u);
        });
    }
}

void launch_logprob(const Launch &L, const uint64_t *chunk_best, double *chunk_sum,
                    const int32_t *tokens, long tokens_ld, int k_per_row, double *out, long out_ld) {
    const dim3 grid(L.rv.n_chunks, L.rows), block(TPB);
    if (L.nv == 8)
        k_chunk_lse<8><<<grid, block, 0, L.stream>>>(L.rv, chunk_best, chunk_sum);
    else
        k_chunk_lse<2><<<grid, block, 0, L.stream>>>(L.rv, chunk_best, chunk_sum);
    k_final_logprob<<<dim3(L.rows), block, 0, L.stream>>>(L.rv, chunk_best, chunk_sum, tokens,
                                                         tokens_ld, k_per_row, out, out_ld);
}

void launch_ngram_draft(hipStream_t stream, const int32_t *history, long history_ld,
                        const int32_t *history_len, const int32_t *seeds, int n_seq, int k_max,
                        int max_suffix, int32_t *out, long out_ld, int32_t *out_count,
                        int32_t *out_match) {
    k_ngram_draft<<<dim3(n_seq), dim3(TPB), 0, stream>>>(history, history_ld, history_len, seeds,
                                                         k_max, max_suffix, out, out_ld, out_count,
                                                         out_match);
}

void launch_penalties(const Launch &L, float *logits_rw) {
    const dim3 grid(L.rv.n_chunks, L.rows), block(TPB);
    if (L.nv == 8)
        k_penalties<8><<<grid, block, 0, L.stream>>>(L.rv, logits_rw);
    else
        k_penalties<2><<<grid, block, 0, L.stream>>>(L.rv, logits_rw);
}

void launch_rng_units(hipStream_t stream, uint64_t *states, int shared, int rows,
                      float *uniforms) {
    const int blocks = shared ? 1 : (rows + 255) / 256;
    k_rng_units<<<dim3(blocks), dim3(shared ? 64 : 256), 0, stream>>>(states, shared, rows,
                                                                      uniforms);
}

} // namespace gs

#ifdef GS_PHASE_STAMPS
/* Instrumented builds only (`make -C geistlib_amd phase-stamps`): the device timestamps that
 * k_cand_scan_final's workgroups took at their phases during the launches so far, 16 per
 * workgroup (sampler_cands_one_launch.h). */
extern "C" int geist_hip_phase_stamps_read(unsigned long long *host, size_t n) {
    return (int) hipMemcpyFromSymbol(host, HIP_SYMBOL(gs::g_phase_stamps),
                                     n * sizeof(unsigned long long));
}
#endif

#ifdef GS_WALK_STAMPS
extern "C" int geist_hip_walk_stamps_read(unsigned long long *host, size_t n) {
    return (int) hipMemcpyFromSymbol(host, HIP_SYMBOL(gs::g_walk_stamps),
                                     n * sizeof(unsigned long long));
}
#endif
