/*
 * sampler_walk_coop.h -- the whole-row walk of the top-p / min-p modes (sampler.c:246-304: sort
 * by probability, keep the nucleus, draw) spread over the workgroups of the row's chunks.
 *
 * One workgroup walking a row of 128 k probabilities makes some nine passes over them, 275 to
 * 300 us in all. Here the workgroup of each chunk keeps its 8192 probabilities in registers, and
 * a pass is: every workgroup adds its share to a histogram of the row in global memory
 * (agent-scope atomics; sums of integers, so their order does not matter), the workgroups meet at
 * the row's arrival counter, the one that arrives last reads the histogram, selects the digit as
 * the one-workgroup walk does (sg_select_digit) and publishes the result with the step's number
 * in one 16-byte record; the others wait for that number. The steps: the first level of the
 * nucleus descent together with the min-p sums, its two further levels, the draw's descent --
 * whose first level is read off the first step's histogram without a meeting
 * (coop_first_level_local), two levels meet --, and the index-order count that finds the j-th
 * entry equal to the drawn value. The histograms take turns, and each is cleared by the waiting
 * workgroups of the meeting after its own (CoopTurn). The arithmetic is that of
 * sorted_descend<false> (sampler_sorted_prob.h) step for step: masses in 2^-62 fixed point, the
 * same targets, the same edge rules.
 *
 * No fences: a workgroup's atomics are acknowledged (s_waitcnt vmcnt(0)) before it arrives, and
 * what the last arrival publishes is written and read with agent-scope accesses. Every wait is
 * bounded (`wait_limit` polls); a workgroup whose wait runs out leaves -- it is then missed at the
 * next meeting, where the others' waits run out in turn --, the row keeps its flag, and the
 * one-workgroup walk that the host launches behind this kernel serves it: a row is always served,
 * whatever the others do. At the last step every workgroup reports how many entries equal to the
 * drawn value its chunk holds, and once all have, the one whose chunk holds the j-th of them in
 * index order writes the token. The row's workspace is zero before the first launch and left zero by every launch that
 * ends without a wait running out (steps are numbered on from `step_base`, so the published
 * number needs no clearing); a launch in which one did says so in the host's hint words (the
 * call's number: in word 0 when a row was walked in full, in word 1 when a wait ran out), and the
 * host clears the workspace before the next.
 */
#ifndef GEIST_SAMPLER_WALK_COOP_H
#define GEIST_SAMPLER_WALK_COOP_H

namespace gs {

constexpr int COOP_HISTS = 4; /* 0: the first step's, kept for the draw; 1..3 take turns */
struct CoopRow {
    uint32_t cnt[COOP_HISTS][SG_BINS];
    uint64_t mass[COOP_HISTS][SG_BINS];
    uint64_t aux[4];                /* sums of the first step, added by every workgroup (three used) */
    uint32_t chunk_cnt[MAX_CHUNKS]; /* entries equal to the drawn value, per chunk */
    /* what a waiting workgroup reads with one 16-byte load: the number of the last step whose
     * result is published, and that result's digit, count above and ties */
    __attribute__((aligned(16))) uint32_t pub[4];
    uint64_t res_mass_above;
    uint32_t arrive;
    uint32_t pad;
};
static_assert(sizeof(CoopRow) % 16 == 0, "rows of the workspace stay 16-byte aligned");
static_assert(offsetof(CoopRow, pub) % 16 == 0, "the published record is one aligned 16-byte load");

__device__ __forceinline__ uint32_t coop_ld32(const uint32_t *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t coop_ld64(const uint64_t *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void coop_st32(uint32_t *p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void coop_st64(uint64_t *p, uint64_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
/* four dwords with one agent-scope load (16-byte aligned: one request, one moment) */
typedef uint32_t coop_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ coop_u32x4 coop_ld128(const uint32_t *p) {
    coop_u32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)"
                 : "=v"(v)
                 : "v"(p)
                 : "memory");
    return v;
}
__device__ __forceinline__ void coop_add32(uint32_t *p, uint32_t v) {
    (void) __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void coop_add64(uint64_t *p, uint64_t v) {
    (void) __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/* Device timestamps of the first row's workgroups, compiled in only with -DGS_WALK_STAMPS. */
#ifdef GS_WALK_STAMPS
__device__ unsigned long long g_walk_stamps[64 * 32];
__device__ __forceinline__ void walk_stamp(int row, int chunk, int i) {
    if (row == 0 && threadIdx.x == 0 && chunk < 64 && i < 32)
        g_walk_stamps[chunk * 32 + i] = wall_clock64();
}
#define GS_WSTAMP(i) walk_stamp(row, chunk, (i))
#else
#define GS_WSTAMP(i) do { } while (0)
#endif

/* pn_fx() for the bits of a probability 0 <= p <= 1 without the trip through double: p * 2^62 is
 * the 24-bit significand shifted by the exponent, truncated as __double2ull_rz truncates (the
 * product is exact in double, so the two agree bit for bit: compared on the host for every
 * binary32 in [0, 1]). */
__device__ __forceinline__ uint64_t pn_fx_bits(uint32_t key) {
    const uint32_t e  = key >> 23; /* (the sign is 0) */
    const uint32_t m  = e ? (key & 0x7fffffu) | 0x800000u : key & 0x7fffffu;
    const int      sh = (int) (e ? e : 1u) - 88; /* value = m * 2^sh, -87 <= sh <= 39 */
    return sh >= 0 ? (uint64_t) m << sh : sh > -24 ? (uint64_t) (m >> -sh) : 0ull;
}

struct CoopShared {
    int      last;   /* this workgroup arrived last at the step's meeting */
    int      ok;     /* the step's result has been published */
    uint32_t pub[4]; /* ... and what was published with it */
};

/* What the workgroup has added to the row's workspace is performed; true in the workgroup that
 * arrives last of the row's W. */
__device__ __forceinline__ bool coop_arrive(CoopRow *cr, int W, CoopShared &cs) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t before =
            __hip_atomic_fetch_add(&cr->arrive, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        cs.last = before == (uint32_t) W - 1u;
        if (cs.last)
            coop_st32(&cr->arrive, 0u); /* (nobody arrives again before the step is published) */
    }
    __syncthreads();
    return cs.last != 0;
}
/* The last arrival's results are written: publish the step. */
__device__ __forceinline__ void coop_publish(CoopRow *cr, uint32_t step) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0)
        coop_st32(&cr->pub[0], step);
}
/* Waits until the step is published; false when the wait ran out. */
__device__ __forceinline__ bool coop_wait(const CoopRow *cr, uint32_t step, uint32_t limit,
                                          CoopShared &cs) {
    if (threadIdx.x == 0) {
        int      ok = 0;
        uint32_t polls = 0;
        for (;;) {
            const coop_u32x4 v = coop_ld128(cr->pub);
            if ((int32_t) (v.x - step) >= 0) {
                /* (the result was written and acknowledged before the number was) */
                cs.pub[1] = v.y, cs.pub[2] = v.z, cs.pub[3] = v.w;
                ok = 1;
                break;
            }
            if (polls++ >= limit)
                break;
            __builtin_amdgcn_s_sleep(2);
        }
        cs.ok = ok;
    }
    __syncthreads();
    const bool ok = cs.ok != 0;
    __syncthreads();
    return ok;
}

/* This workgroup's share of clearing histogram hb (a W-th of its bins). The stores are
 * acknowledged before the workgroup arrives at its next meeting. */
__device__ __forceinline__ void coop_clear_slice(CoopRow *cr, int hb, int chunk, int W) {
    if (hb < 0)
        return;
    const int per = (SG_BINS + W - 1) / W;
    const int end = (chunk + 1) * per < SG_BINS ? (chunk + 1) * per : SG_BINS;
    for (int i = chunk * per + (int) threadIdx.x; i < end; i += TPB) {
        coop_st32(&cr->cnt[hb][i], 0u);
        coop_st64(&cr->mass[hb][i], 0ull);
    }
}

/* The histograms of the steps that meet. The first step's goes to histogram 0, which stays until
 * the draw's first level has been read from it; the others take turns through 1..3. A
 * histogram is cleared by all workgroups, a slice each, while they wait at the NEXT meeting
 * (everyone has read it by then: only the last arrival reads it, before it publishes), and is
 * used again no sooner than three meetings later -- with a meeting in between at which every
 * workgroup's clearing stores are acknowledged. */
struct CoopTurn {
    int hb;     /* this step's histogram */
    int clr[2]; /* histograms to clear while waiting at this step's meeting, or -1 */
};

/* One level of a descent over the row: `add(key)` says whether an entry of this workgroup takes
 * part; its digit is (key >> shf) & dm. With `select` the last arrival picks the digit at which
 * the running mass reaches `target` and publishes it; mass_above / cnt_above / ties are updated
 * in every workgroup. Returns 1 (digit in `digit`), 0 (the target is not reached, or nothing
 * was to be selected), -1 (the wait ran out). */
template <int NK, typename Take>
__device__ __forceinline__ int coop_level(CoopRow *cr, int W, uint32_t &step, uint32_t limit,
                                          SortedGenShared &sh, CoopShared &cs,
                                          const uint32_t (&key)[NK], Take take, int shf,
                                          uint32_t dm, CoopTurn turn, bool select, bool clear_aux,
                                          uint64_t target, uint64_t &mass_above,
                                          uint32_t &cnt_above, uint32_t &ties, int &digit,
                                          int row, int chunk, int sbase) {
    const int tid = threadIdx.x;
    (void) row, (void) sbase;
    for (int i = tid; i < SG_BINS; i += TPB) {
        sh.cnt[i]  = 0u;
        sh.mass[i] = 0ull;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NK; ++i) {
        if (take(key[i])) {
            const uint32_t d = (key[i] >> shf) & dm;
            atomicAdd(&sh.cnt[d], 1u);
            atomicAdd((unsigned long long *) &sh.mass[d], (unsigned long long) pn_fx_bits(key[i]));
        }
        /* (four entries at a time: interleaving all of them costs registers, not time) */
        if ((i & 3) == 3)
            __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
    for (int i = tid; i < SG_BINS; i += TPB) {
        const uint32_t c = sh.cnt[i];
        if (c) {
            coop_add32(&cr->cnt[turn.hb][i], c);
            coop_add64(&cr->mass[turn.hb][i], sh.mass[i]);
        }
    }
    ++step;
    GS_WSTAMP(sbase);
    if (coop_arrive(cr, W, cs)) {
        GS_WSTAMP(sbase + 1);
        {
            /* all of a thread's loads in flight together: one round trip, not sixteen */
            constexpr int PER = SG_BINS / TPB;
            uint32_t      c[PER];
            uint64_t      m[PER];
#pragma unroll
            for (int q = 0; q < PER; ++q)
                c[q] = coop_ld32(&cr->cnt[turn.hb][q * TPB + tid]);
#pragma unroll
            for (int q = 0; q < PER; ++q)
                m[q] = coop_ld64(&cr->mass[turn.hb][q * TPB + tid]);
#pragma unroll
            for (int q = 0; q < PER; ++q) {
                sh.cnt[q * TPB + tid]  = c[q];
                sh.mass[q * TPB + tid] = m[q];
            }
        }
        __syncthreads();
        if (select)
            sg_select_digit(sh, target, mass_above, cnt_above);
        if (tid == 0) {
            const int d = select ? sh.res_digit : -1;
            cs.pub[1] = (uint32_t) d;
            coop_st32(&cr->pub[1], (uint32_t) d);
            if (d >= 0) {
                cs.pub[2] = sh.res_cnt_above, cs.pub[3] = sh.cnt[d];
                coop_st32(&cr->pub[2], sh.res_cnt_above);
                coop_st32(&cr->pub[3], sh.cnt[d]);
                coop_st64(&cr->res_mass_above, sh.res_mass_above);
            }
        }
        coop_publish(cr, step);
        /* (behind the publication: the others are on their way already) */
        if (clear_aux && tid < 4) /* (every workgroup has read them before it arrived here) */
            coop_st64(&cr->aux[tid], 0ull);
        coop_clear_slice(cr, turn.clr[0], chunk, W);
        coop_clear_slice(cr, turn.clr[1], chunk, W);
    } else {
        coop_clear_slice(cr, turn.clr[0], chunk, W);
        coop_clear_slice(cr, turn.clr[1], chunk, W);
        if (!coop_wait(cr, step, limit, cs))
            return -1;
    }
    GS_WSTAMP(sbase + 2);
    /* the digit, the count above and the ties came with the step's number (cs.pub: written by
     * thread 0 before a barrier in either branch); the mass above is loaded now and not needed
     * before the next meeting's selection or the descent's end */
    digit = (int) cs.pub[1];
    if (digit < 0)
        return 0;
    cnt_above  = cs.pub[2];
    ties       = cs.pub[3];
    mass_above = cs.last ? sh.res_mass_above : coop_ld64(&cr->res_mass_above);
    return 1;
}

/* The first level of the draw's descent without a meeting. The first step's histogram (every
 * entry of the row by the leading 11 bits of its key, histogram 0) holds what that level would
 * collect again: the digits above the edge's are the same, those below it are empty, and the
 * edge's own digit holds the entries greater than the edge -- their count and mass, gt_cnt and
 * gt_mass, less those of the digits above -- and the block of limit_ties entries equal to it.
 * Every workgroup reads the histogram and selects for itself (integers: the same result in
 * all). Returns 1 with the digit, or 0 (the target is not reached). */
__device__ __forceinline__ int coop_first_level_local(const CoopRow *cr, SortedGenShared &sh,
                                                      uint64_t target, bool limited,
                                                      uint32_t limit_key, uint32_t limit_ties,
                                                      uint32_t gt_cnt, uint64_t gt_mass,
                                                      uint64_t &mass_above, uint32_t &cnt_above,
                                                      uint32_t &ties, int &digit) {
    const int     tid = threadIdx.x;
    constexpr int PER = SG_BINS / TPB;
    const int     de  = limited ? (int) (limit_key >> 21) : -1;
    uint32_t      c[PER];
    uint64_t      m[PER];
#pragma unroll
    for (int q = 0; q < PER; ++q)
        c[q] = coop_ld32(&cr->cnt[0][q * TPB + tid]);
#pragma unroll
    for (int q = 0; q < PER; ++q)
        m[q] = coop_ld64(&cr->mass[0][q * TPB + tid]);
    uint64_t above_c = 0ull, above_m = 0ull;
#pragma unroll
    for (int q = 0; q < PER; ++q) {
        const int i = q * TPB + tid;
        if (i > de) {
            above_c += c[q];
            above_m += m[q];
        } else {
            c[q] = 0u, m[q] = 0ull;
        }
        sh.cnt[i]  = c[q];
        sh.mass[i] = m[q];
    }
    if (limited) {
        above_c = block_sum_u64(above_c, sh.red64);
        above_m = block_sum_u64(above_m, sh.red64);
        if (tid == 0) {
            sh.cnt[de]  = gt_cnt - (uint32_t) above_c + limit_ties;
            sh.mass[de] = gt_mass - above_m + pn_fx(__uint_as_float(limit_key)) * (uint64_t) limit_ties;
        }
    }
    __syncthreads();
    sg_select_digit(sh, target, 0ull, 0u);
    const int d = sh.res_digit;
    if (d >= 0) {
        mass_above = sh.res_mass_above;
        cnt_above  = sh.res_cnt_above;
        ties       = sh.cnt[d];
    }
    digit = d;
    __syncthreads();
    return d >= 0 ? 1 : 0;
}

/* Three levels (11, 11, 10 bits of the key): sg_descent over the row's workgroups. `lead` is
 * the row's first workgroup, which adds the block of limit_ties entries equal to limit_key.
 * `meet` counts the row's meetings so far (it picks the histograms, see CoopTurn). With
 * `local_first` the first level is coop_first_level_local. `last` is the row's last descent: its
 * last level also clears histogram 0. Returns 1 / 0 / -1 as coop_level. */
template <int NK>
__device__ __forceinline__ int coop_descent(CoopRow *cr, int W, uint32_t &step, uint32_t limit,
                                            SortedGenShared &sh, CoopShared &cs,
                                            const uint32_t (&key)[NK], bool lead, bool clear_aux,
                                            uint64_t target, bool limited, uint32_t limit_key,
                                            uint32_t limit_ties, int &meet, bool local_first,
                                            uint32_t gt_cnt, uint64_t gt_mass, bool last,
                                            uint32_t &kappa, uint32_t &cnt_above,
                                            uint64_t &mass_above, uint32_t &ties_total,
                                            int row, int chunk, int sbase) {
    uint32_t prefix = 0u, mask = 0u;
    cnt_above  = 0u;
    mass_above = 0ull;
    ties_total = 0u;
#pragma unroll 1
    for (int lv = 0; lv < 3; ++lv) {
        const int      shf = lv == 0 ? 21 : lv == 1 ? 10 : 0;
        const uint32_t dm  = lv == 2 ? 1023u : 2047u;
        if (lv == 0 && local_first) {
            int       digit = -1;
            const int r = coop_first_level_local(cr, sh, target, limited, limit_key, limit_ties,
                                                 gt_cnt, gt_mass, mass_above, cnt_above,
                                                 ties_total, digit);
            if (r <= 0)
                return r;
            prefix |= (uint32_t) digit << shf;
            mask |= dm << shf;
            continue;
        }
        /* meeting number `meet` (0 = the row's first): its histogram, and what it clears */
        CoopTurn turn;
        turn.hb     = meet == 0 ? 0 : 1 + (meet - 1) % 3;
        turn.clr[0] = meet >= 2 ? 1 + (meet - 2) % 3 : -1; /* the meeting before, unless the first */
        turn.clr[1] = last && lv == 2 ? 0 : -1;
        ++meet;
        /* the block of entries equal to the limit, as one more key of the first workgroup's
         * first thread: handled apart, its mass is limit_ties times the entry's */
        const bool block_here = limited && lead && threadIdx.x == 0 && limit_ties &&
                                (limit_key & mask) == prefix;
        auto take = [&](uint32_t k) {
            return k != 0xffffffffu && (k & mask) == prefix && !(limited && k <= limit_key);
        };
        /* the block is added after the level's own zeroing: through a key list of one more
         * entry would cost every level a register; it goes straight to the global histogram */
        if (block_here) {
            const uint32_t d = (limit_key >> shf) & dm;
            coop_add32(&cr->cnt[turn.hb][d], limit_ties);
            coop_add64(&cr->mass[turn.hb][d], pn_fx(__uint_as_float(limit_key)) * (uint64_t) limit_ties);
        }
        int       digit = -1;
        const int r = coop_level<NK>(cr, W, step, limit, sh, cs, key, take, shf, dm, turn, true,
                                     clear_aux && lv == (local_first ? 1 : 0), target, mass_above,
                                     cnt_above, ties_total, digit, row, chunk, sbase + 3 * lv);
        if (r <= 0)
            return r;
        prefix |= (uint32_t) digit << shf;
        mask |= dm << shf;
    }
    kappa = prefix;
    return 1;
}

template <int NV, bool PEN>
__global__ __launch_bounds__(TPB, 2) void k_whole_row_coop(RowView rv, SortedRowArgs g, CandSpace cand,
                                                        float top_p, float min_p,
                                                        const float *__restrict__ uniforms,
                                                        int32_t *__restrict__ row_flag,
                                                        int32_t *__restrict__ out,
                                                        CoopRow *__restrict__ coop,
                                                        uint32_t step_base, uint32_t wait_limit,
                                                        uint32_t *__restrict__ hint,
                                                        uint32_t call) {
    __shared__ SortedGenShared sh;
    __shared__ CoopShared      cs;
    __shared__ __align__(16) uint32_t s_cnt16[PEN ? NV * TPB * 2 : 1];
    __shared__ uint64_t s_tab[32];
    __shared__ double   s_total;
    __shared__ int      s_scan[NWAVES];
    int row, chunk;
    xcd_row_chunk(row, chunk);
    if (row_flag[row] != 2)
        return;
    GS_WSTAMP(0);
    const int   tid = threadIdx.x, W = rv.n_chunks;
    const bool  lead = chunk == 0;
    const float u    = uniforms[row];
    CoopRow    *cr   = coop + row;
    if (lead && tid == 0 && hint)
        hint[0] = call; /* rows are being walked in full: the host keeps sending them here */
    /* A row that is not served here keeps its flag, and the one-workgroup walk of the launch
     * behind this one serves it: rows whose sums are not finite (the reference's own answer for
     * those comes out of that walk), and rows of a launch in which a wait ran out -- then the
     * row's workspace may hold a step's remains, and the host is told to clear it. */
    auto alone = [&](bool dirty) {
        if (dirty && lead && tid == 0 && hint)
            hint[1] = call;
    };
    if (tid < 32)
        s_tab[tid] = g_expf_tab[tid];
    if (tid == 0) {
        double t = 0.0;
        for (int c = 0; c < rv.n_chunks; ++c)
            t += g.chunk_sum[(long) row * rv.n_chunks + c];
        s_total = t;
    }
    const float mx = key2f(best_key(row_best_from_chunks(g.chunk_best, row, rv.n_chunks, sh.red64)));
    __syncthreads();
    const double tot = s_total;
    if (!(tot > 0.0 && tot < __builtin_inf() && mx > -__builtin_inff() && mx < __builtin_inff())) {
        alone(false);
        return;
    }
    /* this chunk's normalised probabilities pn = (float)((double)p / sum) (sampler.c:246-253),
     * kept in registers as their bit patterns; 0xffffffff marks places beyond the row */
    int base, end;
    chunk_bounds<NV>(rv, chunk, base, end);
    uint32_t key[4 * NV];
    {
        float4 v[NV];
        fetch_chunk<NV, PEN>(rv, row, rv.n_rows, base, end, s_cnt16, v);
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int e = base + 4 * (j * TPB + tid);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                uint32_t k = 0xffffffffu;
                if (e + c < end) {
                    const float p = geist_expf_glibc_le0(softmax_arg(f4_get(v[j], c), mx, g.inv_t), s_tab);
                    k             = __float_as_uint((float) ((double) p / tot));
                }
                key[4 * j + c] = k;
            }
            /* one group of four at a time: left alone the compiler interleaves all 32
             * evaluations, and the registers that takes cost the kernel its occupancy */
            if (j + 1 < NV)
                asm volatile("" : "+v"(key[4 * j + 3]), "+v"(v[j + 1].x), "+v"(v[j + 1].y),
                                  "+v"(v[j + 1].z), "+v"(v[j + 1].w));
        }
    }
    GS_WSTAMP(1);
    const bool use_p = top_p > 0.0f && top_p < 1.0f;
    const bool use_m = min_p > 0.0f;
    /* the largest probability is that of the row's maximum: expf(0) = 1 over the sum */
    const uint32_t kmax    = __float_as_uint((float) (1.0 / tot));
    const float    floor_w = __fmul_rn(min_p, __uint_as_float(kmax));
    uint32_t       step    = step_base;
    /* ---- step 1: the first level of the nucleus descent; with it the sums that the kept prefix
     * may need: mass and count of the min-p prefix, or the row's mass where no nucleus is asked
     * for ---- */
    if (use_m || !use_p) {
        uint64_t a[4] = {0ull, 0ull, 0ull, 0ull};
#pragma unroll
        for (int i = 0; i < 4 * NV; ++i) {
            if (key[i] == 0xffffffffu)
                continue;
            const uint64_t fx = pn_fx_bits(key[i]);
            if (use_m && __uint_as_float(key[i]) >= floor_w) {
                a[0] += fx;
                a[1] += 1ull;
            }
            a[2] += fx;
            if ((i & 3) == 3)
                __builtin_amdgcn_sched_barrier(0);
        }
        /* the sums over the workgroup with one barrier between them (the histogram's words are
         * free until the first level clears them) */
#pragma unroll
        for (int q = 0; q < 3; ++q)
#pragma unroll
            for (int m = 32; m >= 1; m >>= 1)
                a[q] += shfl_xor_u64(a[q], m);
        if ((tid & (WAVE - 1)) == 0) {
#pragma unroll
            for (int q = 0; q < 3; ++q)
                sh.mass[(tid / WAVE) * 4 + q] = a[q];
        }
        __syncthreads();
        if (tid < 3) {
            uint64_t t = 0;
#pragma unroll
            for (int w = 0; w < NWAVES; ++w)
                t += sh.mass[w * 4 + tid];
            if (t)
                coop_add64(&cr->aux[tid], t);
        }
        __syncthreads();
    }
    GS_WSTAMP(2);
    uint32_t kappa = 0u, cnt_above = 0u, ties = 0u;
    uint64_t mass_above = 0ull;
    const uint64_t target = (uint64_t) __double2ull_ru((double) top_p * 0x1p62);
    int      r, meet = 0;
    {
        /* (the three levels of coop_descent, the first of them also carrying the sums above) */
        r = coop_descent<4 * NV>(cr, W, step, wait_limit, sh, cs, key, lead, false,
                                 use_p ? target : ~0ull, false, 0u, 0u, meet, false, 0u, 0ull,
                                 false, kappa, cnt_above, mass_above, ties, row, chunk, 8);
        if (r < 0) {
            alone(true);
            return;
        }
    }
    GS_WSTAMP(3);
    const uint64_t mass_m = coop_ld64(&cr->aux[0]);
    uint32_t       n_m    = (uint32_t) coop_ld64(&cr->aux[1]);
    const uint64_t mass_all = coop_ld64(&cr->aux[2]);
    uint64_t mass_m_use = mass_m;
    /* the draw's first level can be read off the first step's histogram when the count and mass
     * of the entries above the edge are at hand */
    bool     local_first = true;
    uint32_t gt_cnt = 0u;
    uint64_t gt_mass = 0ull;
    if (use_m && n_m < 1u) {
        n_m         = 1u;
        mass_m_use  = pn_fx(__uint_as_float(kmax));
        local_first = false;
    }
    /* ---- the kept prefix, as sorted_descend<false> decides it ---- */
    bool     limited   = false;
    uint32_t edge_key  = 0u, edge_ties = 0u;
    uint64_t mass_keep = 0ull;
    uint32_t n_keep    = (uint32_t) rv.n_vocab;
    bool     have_p    = false;
    if (use_p && r == 1) {
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
        gt_cnt    = cnt_above;
        gt_mass   = mass_above;
    }
    if (use_m && (!have_p || n_m < n_keep)) {
        limited   = true;
        mass_keep = mass_m_use;
        edge_key  = __float_as_uint(floor_w) ? __float_as_uint(floor_w) - 1u : 0u;
        edge_ties = 0u;
        gt_cnt    = n_m;
        gt_mass   = mass_m_use;
        if (__float_as_uint(floor_w) == 0u)
            limited = false;
    } else if (!have_p) {
        mass_keep = mass_all;
        limited   = false;
    }
    /* ---- the draw ---- */
    const uint64_t target2 = (uint64_t) __double2ull_rd((double) u * (double) mass_keep) + 1ull;
    uint32_t       kd = 0u, cnt_above_d = 0u, ties_d = 0u;
    uint64_t       mass_above_d = 0ull;
    r = coop_descent<4 * NV>(cr, W, step, wait_limit, sh, cs, key, lead, true, target2, limited,
                             edge_key, edge_ties, meet, local_first, gt_cnt, gt_mass, true, kd,
                             cnt_above_d, mass_above_d, ties_d, row, chunk, 17);
    if (r <= 0) { /* 0: not reachable with exact integer masses; the one-workgroup walk decides */
        alone(true);
        return;
    }
    GS_WSTAMP(4);
    const uint64_t each = pn_fx(__uint_as_float(kd));
    uint64_t       j    = each ? (target2 - mass_above_d + each - 1) / each : 1;
    if (j < 1)
        j = 1;
    if (j > ties_d)
        j = ties_d;
    /* ---- the j-th entry, in index order, equal to the drawn value: every workgroup reports how
     * many its chunk holds; once all have, the one whose chunk holds the entry finds it ---- */
    uint32_t here;
    {
        int mine = 0;
#pragma unroll
        for (int i = 0; i < 4 * NV; ++i)
            mine += (int) (key[i] == kd);
        here = (uint32_t) block_sum_u64((uint64_t) mine, sh.red64);
        if (tid == 0)
            coop_st32(&cr->chunk_cnt[chunk], here);
    }
    ++step;
    const int last_hb = 1 + (meet - 2) % 3; /* (the draw's last level met: meet >= 3) */
    if (coop_arrive(cr, W, cs)) {
        GS_WSTAMP(5);
        coop_publish(cr, step);
        coop_clear_slice(cr, last_hb, chunk, W);
    } else {
        coop_clear_slice(cr, last_hb, chunk, W);
        if (!coop_wait(cr, step, wait_limit, cs)) {
            alone(true);
            return;
        }
    }
    /* the entries in the chunks before this one (a thread per chunk, then their sum) */
    const uint64_t before =
        block_sum_u64(tid < chunk ? (uint64_t) coop_ld32(&cr->chunk_cnt[tid]) : 0ull, sh.red64);
    if (!(before < j && j <= before + here))
        return; /* the entry lies in another chunk */
    int want = (int) (j - before); /* 1-based, among the chunk's entries in index order */
#pragma unroll
    for (int q = 0; q < NV; ++q) { /* a chunk's index order: group q, then thread, then element */
        const int m_q = (int) (key[4 * q] == kd) + (int) (key[4 * q + 1] == kd) +
                        (int) (key[4 * q + 2] == kd) + (int) (key[4 * q + 3] == kd);
        int       total;
        const int incl = block_scan_i32(m_q, s_scan, &total);
        if (want >= 1 && want <= total && incl >= want && incl - m_q < want) {
            int seen = incl - m_q;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if (key[4 * q + c] == kd && ++seen == want) {
                    out[row]       = base + 4 * (q * TPB + tid) + c;
                    cand.path[row] = 4;
                    row_flag[row]  = 0; /* served */
                }
            }
        }
        want -= total; /* (at or below zero once found: no later group matches) */
    }
    GS_WSTAMP(6);
}

} // namespace gs
#endif
