/*
 * sampler_cands_one_launch.h -- the top-k path (sampler.c:178-228, with penalties, soft-cap,
 * top-p and min-p of the chain) as ONE launch, for batches that fit the device at one workgroup of
 * 1024 threads per compute unit.
 *
 *   k_cand_scan_final   G = ceil(chunks / 4) workgroups per row; the grid holds the rows in
 *                       eights so that the workgroups of a row have linear ids equal modulo 8,
 *                       which this device places on one XCD (workgroups of rows that are not
 *                       there leave at once). A workgroup holds 32768 logits of its row in
 *                       registers (a wavefront 2048, a lane 32 in eight groups of four; in
 *                       launches of few rows half of that, NG = 4, so that twice the compute
 *                       units fetch a row). It
 *                       finds a bound T_w that about r of its group maxima reach, hands on the
 *                       groups whose maximum reaches T_w -- a few dozen (float4, index) pairs,
 *                       in slots of their own per wavefront -- and adds itself to the row's
 *                       arrival counter. The workgroup that arrives last goes on as the row's
 *                       final stage: B = the largest T_w of the row; every element of the row at
 *                       or above B was handed on by its workgroup (each handed on every group
 *                       with an element >= its own T_w <= B). If k of them still reach B after
 *                       the penalties, the row's k largest are among them (sampler.c:202-215
 *                       keeps the k largest of the sorted row): they are ordered by counting
 *                       (logit descending, index ascending: sampler.c:207 with a stable sort) and
 *                       the first wavefront finishes (softmax over the k, top-p, min-p, draw).
 *                       A row that cannot be certified this way -- leading logits crowded into
 *                       one workgroup, runs of equal values, rows of -inf, many penalised
 *                       leaders, more groups than slots -- forms its thread maxima and takes the
 *                       slower exact paths inside the same launch.
 *
 * `r` is chosen on the host so that a workgroup holding r of the row's k leading logits is a
 * one-in-10^8 event for logits whose order is unrelated to the vocabulary order (r_last for the
 * row's last workgroup, which may hold fewer elements); it only decides how often the slower
 * paths run, never the token.
 *
 * What does not depend on the logits is done while their loads are in flight: the row's history
 * is entered into an open-addressing table in LDS (16384 slots: token id and a 16-bit count),
 * the uniform and the expf table are fetched, the lists cleared. The final stage then penalises a
 * candidate after one probe of the table; only candidates are ever penalised (penalties that can
 * only lower a logit leave the bound B valid: the check that k entries still reach B proves that
 * nothing outside the hand-over belongs to the k largest).
 *
 * The hand-over between the workgroups of a row goes through plain stores: the wavefront that
 * wrote its slots waits for their acknowledgement (they are then in the XCD's second-level
 * cache), and the workgroup's last wavefront adds the workgroup to the row's counter with one
 * agent-scope atomic. The sum carries the XCD number of every arrival (count, sum and sum of
 * squares), so the last arrival knows whether all of the row ran on its own XCD: then the slots
 * are in the L2 it shares with them and it reads them with ordinary loads after invalidating its
 * first-level cache. Otherwise (or when the host asks for it, for tests) the hand-over is not
 * read at all: the row takes the slower paths, which read the logits only. Where a row's
 * workgroups are placed can cost time, never a token.
 *
 * With a word in page-locked memory to report to (Notify), the row that completes the batch
 * publishes the call's number there, after every row's id has been written through to `out`.
 */
#ifndef GEIST_SAMPLER_CANDS_ONE_LAUNCH_H
#define GEIST_SAMPLER_CANDS_ONE_LAUNCH_H

namespace gs {

/* Device timestamps of the kernel's phases, compiled in only with -DGS_PHASE_STAMPS (a build for
 * looking at where the time goes; the library as shipped has none of it). */
#ifdef GS_PHASE_STAMPS
__device__ unsigned long long g_phase_stamps[4096 * 16];
#ifndef GS_PHASE_STAMP_MASK
#define GS_PHASE_STAMP_MASK 0xffff /* which of the stamps are taken (each costs its wavefront time) */
#endif
#define GS_STAMP(i)                                                                            \
    do {                                                                                       \
        if (((GS_PHASE_STAMP_MASK) >> (i)) & 1)                                                \
            if (threadIdx.x == 0)                                                              \
                g_phase_stamps[(blockIdx.y * gridDim.x + blockIdx.x) * 16 + (i)] =             \
                    wall_clock64();                                                            \
    } while (0)
#else
#define GS_STAMP(i) do { } while (0)
#endif

constexpr int OL_THREADS = 1024;
constexpr int OL_WAVES   = OL_THREADS / WAVE;
constexpr int OL_N_MAX   = 512; /* entries of a row the final stage orders */
constexpr int OL_N_PAD   = 64;  /* zeros behind the list, for reads in strides */
constexpr int OL_HT_SLOTS = 16384;    /* slots of the history table */
constexpr int OL_HISTORY_MAX = 12288; /* longest history entered into it */
static_assert(OL_WAVES * OL_TOP == 2 * WAVE, "two entered maxima per lane in the bound search");
static_assert(OL_SLOTS == 16 && OL_WAVES == 16, "thread t reads slot t % 16 of wavefront t / 16");
static_assert(OL_WG_MAX * OL_WAVES == 2 * WAVE, "two scanning wavefronts' counts per lane");

struct OneLaunchShared {
    uint32_t tw;      /* key of the workgroup's bound */
    int      ticket;  /* ... whose hand-over has been acknowledged */
    int      n_c;     /* entries of the row's list */
    int      give_up; /* the row cannot be served here */
    int      last;    /* this workgroup arrived last at the row's counter */
    int      far;     /* ... and not all of the row ran on its XCD */
};

/* All lanes receive the number of wavefronts of the workgroup that called before this one. What
 * the earlier callers wrote to LDS before their call is visible after it (the LDS operations of a
 * workgroup are performed in the order they were issued). `counter` must hold zero, published by a
 * barrier, before the first call. */
__device__ __forceinline__ int wave_ticket(int *counter) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    int ticket = 0;
    if ((threadIdx.x & (WAVE - 1)) == 0)
        ticket = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    ticket = (int) readlane_u32((uint32_t) ticket, 0);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    return ticket;
}

__device__ __forceinline__ uint32_t ol_hash(int id) {
    return ((uint32_t) id * 0x9E3779B1u) >> 18; /* 14 bits: OL_HT_SLOTS slots */
}
static_assert(OL_HT_SLOTS == 1 << 14, "ol_hash");

/* The maxima of a thread's eight float4 groups of chunk `chunk` (loaded into v) and their
 * maximum, NaN for a thread whose first element lies beyond the row: what k_cand_scan stores as
 * the thread maximum. */
template <int NG>
__device__ __forceinline__ float group_maxima(const float4 (&v)[NG], float (&gm)[NG], int base,
                                              int end, int t) {
    static_assert(NG == 8 || NG == 4, "eight or four groups a lane");
#pragma unroll
    for (int j = 0; j < NG; ++j)
        gm[j] = max3f(max3f(v[j].x, v[j].y, v[j].z), v[j].w, v[j].w);
    float tm = max3f(gm[0], gm[1], gm[2]);
    if (NG == 8) {
        tm = max3f(tm, gm[3], gm[4]);
        tm = max3f(tm, gm[5], gm[6]);
        tm = max3f(tm, gm[NG - 1], gm[NG - 1]);
    } else {
        tm = max3f(tm, gm[3], gm[3]);
    }
    if (base + 4 * t >= end)
        tm = __builtin_nanf("");
    return tm;
}

/* NG: float4 groups a lane holds, 8 (a workgroup scans 32768 logits) or, for launches of few
 * rows, 4 (16384: twice the workgroups to a row, so that twice the compute units fetch it). */
template <bool PEN, bool STREAM, int NG>
__global__ __launch_bounds__(OL_THREADS) void k_cand_scan_final(RowView rvs, RowView rv,
                                                                WgCands wc, int r_w, int r_last,
                                                                FinalArgs a,
                                                                float *__restrict__ tmax_rw,
                                                                uint32_t *__restrict__ arrive,
                                                                int far_always, Notify nt) {
    /* the table of the row's history (PEN): OL_HT_SLOTS ids and as many 16-bit counters */
    constexpr int ARENA_HT = PEN ? OL_HT_SLOTS * 6 : 16;
    constexpr int ARENA = ARENA_HT > FallbackArena<8, PEN>::END ? ARENA_HT
                                                                : FallbackArena<8, PEN>::END;
    __shared__ __align__(16) uint8_t s_arena[ARENA];
    __shared__ uint64_t        s_tab[32];
    __shared__ uint64_t        s_pack[TOPK_FAST_MAX];
    __shared__ __align__(16) uint64_t s_c[OL_N_MAX + OL_N_PAD];
    __shared__ uint32_t        s_top[OL_WAVES * OL_TOP];
    __shared__ GeneralShared   s_gs;
    __shared__ OneLaunchShared s_o;
    __shared__ int             s_n, s_n2;
    static_assert(TOPK_FAST_MAX == OL_WAVES * OL_TOP, "cleared together");

    const int tid = threadIdx.x, lane = tid & (WAVE - 1);
    const int wv  = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int G   = (int) gridDim.x; /* workgroups per row */
    /* the grid holds the rows in eights: the workgroups of a row have linear ids equal modulo 8 */
    const int lin = (int) (blockIdx.y * gridDim.x + blockIdx.x), slot = lin >> 3;
    const int row = (lin & 7) + 8 * (slot / G), grp = slot % G;
    if (row >= rv.n_rows)
        return; /* the grid's padding */
    int      *hkey = reinterpret_cast<int *>(s_arena);                    /* -1 = empty */
    uint32_t *hcnt = reinterpret_cast<uint32_t *>(s_arena + OL_HT_SLOTS * 4); /* two a word */
    GS_STAMP(0);

    /* ---- everything that does not depend on the logits, asked for before them (loads return in
     * the order they were issued: these can be waited for while the logits are still on their
     * way). Vector loads throughout: a scalar load shares its counter with the LDS traffic. */
    int vz = 0;
    asm volatile("" : "+v"(vz));
    int            hid0 = -1, hid1 = -1, hlen = 0;
    const int32_t *hrow = nullptr;
    if (PEN) {
        hrow = rv.hist + (long) row * rv.hist_ld;
        hlen = rv.hist_len[row + vz];
        if (tid < rv.hist_ld)
            hid0 = hrow[tid];
        if (tid + OL_THREADS < rv.hist_ld)
            hid1 = hrow[tid + OL_THREADS];
    }
    const float u_row = a.uniforms[row + vz];
    uint64_t    tabv  = 0;
    if (tid < 32)
        tabv = g_expf_tab[tid];

    /* ---- the logits: chunk 4 grp + tid / 256, as thread tid % 256 of k_cand_scan holds it. One
     * straight run of eight loads whatever the chunk: a float4 group beyond the row (the row's
     * last chunk, a chunk the row does not have) reads the row's last group instead and is set
     * to -inf afterwards. (A second code path for partial chunks would make the loads of both
     * wait for everything asked for before.) Rows are 16-byte aligned and n_vocab a multiple of
     * four on this path. */
    constexpr int PIECE = NG * TPB * 4; /* what 256 threads hold: a chunk of the scan, or half */
    const int piece = 4 * grp + (tid >> 8), t = tid & (TPB - 1);
    int       base = rvs.n_vocab, end = rvs.n_vocab; /* a piece beyond the row: nothing but -inf */
    if ((long) piece * PIECE < (long) rvs.n_vocab) {
        base = piece * PIECE;
        end  = base + PIECE < rvs.n_vocab ? base + PIECE : rvs.n_vocab;
    }
    const int g0 = (base >> 2) + t, g_last = (rvs.n_vocab >> 2) - 1;
    float4    v[NG];
    {
        const float4 *row4 = reinterpret_cast<const float4 *>(rvs.logits + (long) row * rvs.ld);
#pragma unroll
        for (int j = 0; j < NG; ++j) {
            const int g = g0 + j * TPB;
            v[j] = STREAM ? load_streaming(row4 + (g < g_last ? g : g_last))
                          : row4[g < g_last ? g : g_last];
        }
    }

    /* ---- in the shadow of those loads */
    if (PEN) {
        static_assert(OL_HT_SLOTS % (4 * OL_THREADS) == 0, "whole 16-byte pieces per thread");
#pragma unroll
        for (int i = 0; i < OL_HT_SLOTS / 4 / OL_THREADS; ++i)
            reinterpret_cast<uint4 *>(hkey)[tid + i * OL_THREADS] = make_uint4(~0u, ~0u, ~0u, ~0u);
#pragma unroll
        for (int i = 0; i < OL_HT_SLOTS / 8 / OL_THREADS; ++i)
            reinterpret_cast<uint4 *>(hcnt)[tid + i * OL_THREADS] = make_uint4(0u, 0u, 0u, 0u);
    }
    if (tid < OL_WAVES * OL_TOP) {
        s_top[tid]  = 0u;
        s_pack[tid] = 0ull;
    }
    if (tid < OL_N_MAX + OL_N_PAD)
        s_c[tid] = 0ull;
    if (tid < 32)
        s_tab[tid] = tabv;
    if (tid == 0) {
        s_o.ticket  = 0;
        s_o.n_c     = 0;
        s_o.give_up = 0;
        s_o.last    = 0;
        s_o.far     = 0;
    }
    lds_barrier();
    /* an id of the history takes a slot of the table, or finds it taken by the same id, and
     * counts there (16-bit counters: a history holds fewer than 65536 ids). A history too long
     * for the table is not entered at all: `table_ok` false makes the row take the slower paths. */
    auto enter_id = [&](int id) {
        uint32_t h = ol_hash(id);
#pragma unroll 1
        for (int pr = 0; pr < OL_HT_SLOTS; ++pr) {
            const int old = atomicCAS(&hkey[h], -1, id);
            if (old == -1 || old == id)
                break;
            h = (h + 1u) & (OL_HT_SLOTS - 1);
        }
        atomicAdd(&hcnt[h >> 1], 1u << (16 * (h & 1u)));
    };
    bool table_ok = true;
    if (PEN) {
        hlen     = hlen > rv.hist_ld ? (int) rv.hist_ld : hlen;
        table_ok = hlen <= OL_HISTORY_MAX;
        if (table_ok) {
            if (tid < hlen && (unsigned) hid0 < (unsigned) rv.n_vocab)
                enter_id(hid0);
            if (tid + OL_THREADS < hlen && (unsigned) hid1 < (unsigned) rv.n_vocab)
                enter_id(hid1);
        }
    }
    GS_STAMP(1);

    /* ---- the lane maxima; the largest of every eight neighbouring lanes is entered for the
     * workgroup's bound (three row shifts: lane 8 i + 7 ends with the maximum of its eight) */
    if (ballot64(g0 + (NG - 1) * TPB > g_last) != 0ull) { /* a wavefront at the row's end */
#pragma unroll
        for (int j = 0; j < NG; ++j) {
            const bool out = g0 + j * TPB > g_last;
            v[j].x         = out ? -INFINITY : v[j].x;
            v[j].y         = out ? -INFINITY : v[j].y;
            v[j].z         = out ? -INFINITY : v[j].z;
            v[j].w         = out ? -INFINITY : v[j].w;
        }
    }
    float gm[NG];
    const float tm = group_maxima<NG>(v, gm, base, end, t);
    {
        uint32_t m8 = f2key(tm);
        GS_STAMP(2);
#define GS_STEP(ctrl)                                                                          \
    {                                                                                          \
        const uint32_t o = dpp_fetch_u32<ctrl, 0xf>(m8);                                       \
        m8               = o > m8 ? o : m8;                                                    \
    }
        GS_STEP(0x111) GS_STEP(0x112) GS_STEP(0x114)
#undef GS_STEP
        /* (made distinct: the low seven bits give way to the slot's number, the first slot the
         * greatest -- the bound keeps sixteen leading bits only) */
        if ((lane & 7) == 7) {
            const uint32_t slot = (uint32_t) (wv * OL_TOP + (lane >> 3));
            s_top[slot]         = (m8 & ~127u) | (127u - slot);
        }
    }
    lds_barrier();
    /* T_w: sixteen leading key bits of the r-th largest of the 128 entered maxima (at least r lane
     * maxima reach it). Every wavefront ranks the eight it entered itself: a lane holds two of the
     * 128, an entry travels as a scalar, and two ballots count the entries above it; the entry of
     * rank r - 1 is it. A workgroup with fewer than r maxima -- a few elements at the row's end --
     * finds an empty entry there and hands on all it has. */
    {
        const uint32_t sa = s_top[lane], sb = s_top[lane + WAVE];
        const uint32_t own = wv < OL_WAVES / 2 ? sa : sb;
        const int      r = grp == G - 1 ? r_last : r_w; /* the row's last workgroup holds less */
        uint32_t       found = 0u;
#pragma unroll
        for (int e = 0; e < OL_TOP; ++e) {
            const uint32_t x = readlane_u32(own, (wv & (OL_WAVES / 2 - 1)) * OL_TOP + e);
            const int      c = __popcll(ballot64(sa > x)) + __popcll(ballot64(sb > x));
            found            = c == r - 1 ? (x | 1u) : found; /* (never 0 when found) */
        }
        if (found != 0u && lane == 0) {
            const uint32_t q16 = found & 0xffff0000u;
            /* never below the lowest finite value: -inf (padding, forbidden tokens) is not
             * handed on */
            s_o.tw = q16 < KEY_LOWEST_FINITE ? KEY_LOWEST_FINITE : q16;
        }
    }
    lds_barrier();
    const uint32_t tw = s_o.tw;
    const float    Tf = key2f(tw);
    GS_STAMP(3);
    /* ---- hand-over. Each wavefront writes its float4 groups that hold an element at or above T_w
     * into its own OL_SLOTS slots (places from ballots and lane counts: no atomics), with the
     * index of each group's first element, and their number; more than OL_SLOTS: the row cannot
     * be certified. The first wavefront adds T_w. */
    {
        const long sw  = ((long) row * G + grp) * OL_WAVES + wv; /* this scanning wavefront */
        /* slot p of this wavefront lies at [row][p][wavefront of the row]: the final stage reads
         * one slot of all the row's wavefronts at a time */
        const int  Wr  = G * OL_WAVES;
        float4    *dv  = wc.val + (long) row * OL_SLOTS * Wr + grp * OL_WAVES + wv;
        uint32_t  *di  = wc.idx + (long) row * OL_SLOTS * Wr + grp * OL_WAVES + wv;
        const int  e0  = base + 4 * t;
        unsigned   cnt = 0;
#pragma unroll
        for (int j = 0; j < NG; ++j) {
            const bool     in_j = gm[j] >= Tf;
            const uint64_t mj   = ballot64(in_j);
            if (mj == 0ull)
                continue;
            const unsigned p = cnt + lanes_before(mj);
            if (in_j && p < (unsigned) OL_SLOTS) {
                dv[p * Wr] = v[j];
                di[p * Wr] = (uint32_t) (e0 + 4 * j * TPB);
            }
            cnt += (unsigned) __popcll(mj);
        }
        /* the number of groups (more than OL_SLOTS: too many) beside the sixteen leading bits of
         * T_w, which are all it has */
        if (lane == 0)
            wc.count[sw] = tw | (cnt < 0xffffu ? cnt : 0xffffu);
    }
    if (PEN && table_ok && hlen > 2 * OL_THREADS) { /* a long history: the rest of it */
        for (int i = tid + 2 * OL_THREADS; i < hlen; i += OL_THREADS) {
            const int id = hrow[i];
            if ((unsigned) id < (unsigned) rv.n_vocab)
                enter_id(id);
        }
    }
    GS_STAMP(4);
    /* every wavefront waits for its own stores to be acknowledged and takes a ticket; the one
     * that draws the last adds the workgroup to the row's counter */
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    GS_STAMP(5);
    if (wave_ticket(&s_o.ticket) == OL_WAVES - 1) {
        if (lane == 0) {
            /* hwreg 20 (XCC_ID), bits 3:0 */
            const uint32_t x   = (uint32_t) __builtin_amdgcn_s_getreg(((4 - 1) << 11) | (0 << 6) | 20);
            const uint32_t add = 1u + (x << 8) + ((x * x) << 16);
            uint32_t      *ctr = arrive + (long) row * ARRIVE_STRIDE_INTS;
            const uint32_t tot =
                __hip_atomic_fetch_add(ctr, add, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + add;
            if ((tot & 0xffu) == (uint32_t) G) {
                __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                /* all G numbers equal x  <=>  their sum is G x and the sum of squares G x^2 */
                const bool same = ((tot >> 8) & 0xffu) == (uint32_t) G * x &&
                                  (tot >> 16) == (uint32_t) G * x * x;
                s_o.far  = !same;
                s_o.last = 1;
            }
        }
    }
    GS_STAMP(6);
    __syncthreads();
    if (!s_o.last)
        return;
    GS_STAMP(7);

    /* ================= the row's final stage ================================================= */
    /* Not all of the row on this XCD (or the caller asks for that branch): what the others
     * wrote may still sit in another XCD's cache. The row is then served from the logits alone. */
    const bool far = s_o.far != 0 || far_always != 0;
    asm volatile("buffer_inv sc0" ::: "memory"); /* the first-level cache only */
    /* Every load of the hand-over is issued before any is waited for. The row was scanned by
     * W = 16 G wavefronts; wavefront w of this workgroup takes slot w of every scanning wavefront,
     * lane l that of scanning wavefront l (and 64 + l where the row has more than four
     * workgroups): the wavefronts whose slot no scanning wavefront filled -- most of them --
     * have nothing to do. */
    const int  W = G * OL_WAVES;
    const long sw0 = (long) row * W;
    float4     gv[2];
    uint32_t   gi[2], cw[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const bool on = h == 0 || G > 4;
        const int  w  = lane + 64 * h < W ? lane + 64 * h : 0;
        gv[h] = make_float4(0.f, 0.f, 0.f, 0.f);
        gi[h] = 0u;
        cw[h] = 0u;
        if (on) {
            gv[h] = wc.val[((long) row * OL_SLOTS + wv) * W + w];
            gi[h] = wc.idx[((long) row * OL_SLOTS + wv) * W + w];
            cw[h] = wc.count[sw0 + w]; /* how many groups that scanning wavefront handed on */
        }
        cw[h] = lane + 64 * h < W ? cw[h] : 0u;
    }
    /* B: the largest T_w of the row (each scanning wavefront wrote its workgroup's beside its
     * count) */
    const uint32_t bk = wave_max_u32((cw[0] > cw[1] ? cw[0] : cw[1]) & 0xffff0000u);
    cw[0] &= 0xffffu;
    cw[1] &= 0xffffu;
    const uint32_t lo = bk < KEY_LOWEST_FINITE ? KEY_LOWEST_FINITE : bk;
    GS_STAMP(8);
    const float    B  = key2f(lo);
    /* With the soft-cap left to this stage (FinalArgs::cap_after) an entry counts when its capped
     * value lies strictly above the capped bound: those are certain to be all there are. */
    const float Bc = a.cap_after ? softcap1(B, rv.softcap) : B;
    auto key_of = [&](float x) -> uint32_t { /* 0: the entry no longer counts */
        if (!(x >= B))
            return 0u;
        if (a.cap_after) {
            const float xc = softcap1(x, rv.softcap);
            return xc > Bc ? f2key(xc) : 0u;
        }
        return f2key(x);
    };
    /* a scanning wavefront with more groups than slots, a history the table does not hold, a row
     * spread over XCDs: the row cannot be served here */
    if (ballot64(cw[0] > (uint32_t) OL_SLOTS || cw[1] > (uint32_t) OL_SLOTS) != 0ull || !table_ok || far)
        s_o.give_up = 1; /* (every writer writes 1) */
    /* entry (x, id) into place p of the list, penalised by how often the row's history names
     * the id: looked up in the table (nearly always the first slot tried says no) */
    auto enter = [&](int p, float x, uint32_t id) {
        if (PEN) {
            uint32_t h = ol_hash((int) id);
            int      k = hkey[h];
#pragma unroll 1
            for (int pr = 0; pr < OL_HT_SLOTS && k != (int) id && k != -1; ++pr) {
                h = (h + 1u) & (OL_HT_SLOTS - 1);
                k = hkey[h];
            }
            if (k == (int) id) {
                const uint32_t times = (hcnt[h >> 1] >> (16 * (h & 1u))) & 0xffffu;
                x = penalise(x, times, rv.rep, rv.inv_rep, rv.freq, rv.pres);
            }
        }
        if (p < OL_N_MAX)
            s_c[p] = pack_best(key_of(x), id);
    };
    /* The list of the row: the elements at or above B, in any order (the ranking below orders
     * them). A group's largest element is placed by its wavefront -- which asks for as many
     * places as it has such groups, one atomic a wavefront --; further elements of a group that
     * reach B, few groups have one, ask for a place each. */
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        if (h == 1 && G <= 4)
            break;
        /* the largest of the group (the first of equals) */
        const float x4[4] = {gv[h].x, gv[h].y, gv[h].z, gv[h].w};
        int         cb = 0;
        float       xb = x4[0];
#pragma unroll
        for (int c = 1; c < 4; ++c) {
            const bool up = x4[c] > xb || xb != xb;
            cb            = up ? c : cb;
            xb            = up ? x4[c] : xb;
        }
        const bool     keep = wv < (int) cw[h] && xb >= B;
        const uint64_t mk   = ballot64(keep);
        if (mk == 0ull)
            continue;
        int at = 0;
        if (lane == 0)
            at = atomicAdd(&s_o.n_c, (int) __popcll(mk));
        at = (int) readlane_u32((uint32_t) at, 0) + (int) lanes_before(mk);
        GS_STAMP(12);
        if (keep) {
            enter(at, xb, gi[h] + (uint32_t) cb);
            const int more = (int) (x4[0] >= B) + (int) (x4[1] >= B) + (int) (x4[2] >= B) + (int) (x4[3] >= B);
            if (more > 1) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    if (c != cb && x4[c] >= B)
                        enter(atomicAdd(&s_o.n_c, 1), x4[c], gi[h] + (uint32_t) c);
                }
            }
        }
    }
    GS_STAMP(13);
    __syncthreads();
    GS_STAMP(9);
    const int n_c     = s_o.n_c;
    bool      give_up = s_o.give_up != 0 || n_c > OL_N_MAX;
    if (!give_up) {
        /* Order by counting. A thread counts, for R entries of the list, how many of its share of
         * the list are greater; P neighbouring lanes share the list and a row of DPP shifts adds
         * their counts up. R = 2, P = 16 for up to 128 entries (every thread has work), R = 4 for
         * up to 256, R = 4 and P = 8 beyond: every entry read from LDS is compared R times, and
         * what limits this step is the LDS, then the number of instructions of a thread. The
         * first k that still count are the row's top k. Wavefronts beyond the list have nothing
         * to do. (The list is followed by zeros -- cleared at the start, never written --, which
         * no entry is below: reads may run past its end.) */
        const ulonglong2 *pairs = reinterpret_cast<const ulonglong2 *>(s_c);
        const int         n2    = (n_c + 1) >> 1;
        auto reduce_and_place = [&](int c, uint64_t me, int i, int lp, int part) {
            c += __builtin_amdgcn_update_dpp(0, c, 0x111, 0xf, 0xf, false); /* row_shr:1 */
            c += __builtin_amdgcn_update_dpp(0, c, 0x112, 0xf, 0xf, false); /* row_shr:2 */
            c += __builtin_amdgcn_update_dpp(0, c, 0x114, 0xf, 0xf, false); /* row_shr:4 */
            if (lp == 4)
                c += __builtin_amdgcn_update_dpp(0, c, 0x118, 0xf, 0xf, false); /* row_shr:8 */
            /* (with P = 8 the sums of lanes 0-7 reach lane 7, those of lanes 8-15 lane 15) */
            if (part == (1 << lp) - 1 && i < n_c && best_key(me) != 0u && c < a.k)
                s_pack[c] = me;
        };
        if (n_c <= 128) {
            const int b = tid >> 4, part = tid & 15;
            if ((tid & ~(WAVE - 1)) < (((n_c + 1) >> 1) << 4)) {
                const ulonglong2 m01 = pairs[b];
                int              r0 = 0, r1 = 0;
#pragma unroll 1
                for (int j2 = part; j2 < n2; j2 += 32) {
                    const ulonglong2 q0 = pairs[j2], q1 = pairs[j2 + 16];
                    r0 += (int) (q0.x > m01.x) + (int) (q0.y > m01.x) + (int) (q1.x > m01.x) + (int) (q1.y > m01.x);
                    r1 += (int) (q0.x > m01.y) + (int) (q0.y > m01.y) + (int) (q1.x > m01.y) + (int) (q1.y > m01.y);
                }
                GS_STAMP(14);
                reduce_and_place(r0, m01.x, 2 * b, 4, part);
                reduce_and_place(r1, m01.y, 2 * b + 1, 4, part);
            }
        } else {
            const int lp = n_c <= 256 ? 4 : 3, P = 1 << lp;
            const int b = tid >> lp, part = tid & (P - 1);
            if ((tid & ~(WAVE - 1)) < (((n_c + 3) >> 2) << lp)) {
                const ulonglong2 m01 = pairs[2 * b], m23 = pairs[2 * b + 1];
                const uint64_t   me[4] = {m01.x, m01.y, m23.x, m23.y};
                int              rank[4] = {0, 0, 0, 0};
#pragma unroll 1
                for (int j2 = part; j2 < n2; j2 += 2 * P) {
                    const ulonglong2 q0 = pairs[j2], q1 = pairs[j2 + P];
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        rank[r] += (int) (q0.x > me[r]) + (int) (q0.y > me[r]) + (int) (q1.x > me[r]) +
                                   (int) (q1.y > me[r]);
                }
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    reduce_and_place(rank[r], me[r], 4 * b + r, lp, part);
            }
        }
    }
    GS_STAMP(15);
    __syncthreads();
    GS_STAMP(10);
    /* fewer than k at or above B: B certifies nothing */
    give_up = give_up || s_pack[a.k - 1] == 0ull;
    int k   = a.k;
    if (give_up) {
        /* the thread maxima of the row, as k_cand_scan stores them, for the slower paths (which
         * are written for 256 threads) */
        for (int c = tid >> 8; c < rvs.n_chunks; c += OL_THREADS / TPB) {
            int b2, e2;
            chunk_bounds<8>(rvs, c, b2, e2);
            float4 v2[8];
            float  gm2[8];
            load_raw<8>(rvs, rvs.logits + (long) row * rvs.ld, b2, e2, v2, t);
            tmax_rw[((long) row * rvs.n_chunks + c) * TPB + t] = group_maxima<8>(v2, gm2, b2, e2, t);
        }
        __syncthreads();
        if (tid >= TPB)
            return;
        k = cand_fallback<8, PEN>(&rv, &a, row, s_arena, s_pack, &s_gs, &s_n, &s_n2);
    } else {
        if (tid >= WAVE)
            return;
        if (a.row_flag && tid == 0)
            a.row_flag[row] = 0;
    }
    if (tid < WAVE) {
        /* (k <= CAND_K_MAX = 64 on this path) */
        const int tok = finish_sorted_lanes(k, s_pack, a.inv_t, a.top_p, a.min_p, u_row, s_tab);
        if (tid == 0) {
            if (!nt.h_done) {
                a.out[row] = tok;
            } else {
                /* The id is written through to where `out` lies (a plain store may stay in the
                 * second-level cache until the kernel ends, and the host, told by the word below,
                 * would read the id of the call before) and has arrived before the row counts as
                 * done; the row that completes the batch tells the host. */
                __hip_atomic_store(a.out + row, tok, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                const uint32_t done = __hip_atomic_fetch_add(nt.rows_done, 1u, __ATOMIC_RELAXED,
                                                             __HIP_MEMORY_SCOPE_AGENT) + 1u;
                if (done == (uint32_t) rv.n_rows) {
                    __hip_atomic_store(nt.rows_done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(nt.h_done, nt.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                }
            }
        }
    }
    GS_STAMP(11);
}

/* Writes, per workgroup of a (gx, gy) grid of 1024 threads, the number of the XCD it runs on:
 * whether workgroups with linear ids equal modulo 8 share an XCD decides if the one-launch form
 * is the faster one on a device. */
__global__ __launch_bounds__(OL_THREADS) void k_xcd_of_workgroups(int32_t *__restrict__ out) {
    if (threadIdx.x == 0) /* hwreg 20 (XCC_ID), bits 3:0 */
        out[blockIdx.y * gridDim.x + blockIdx.x] =
            (int32_t) __builtin_amdgcn_s_getreg(((4 - 1) << 11) | (0 << 6) | 20);
}

} // namespace gs
#endif
