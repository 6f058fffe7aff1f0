/*
 * sampler_cands.h -- the top-k path whose single pass over the logits hands candidates on.
 *
 *   k_cand_scan    grid (chunks, rows). A wavefront holds 64 x 4*NV elements of its row. It finds
 *                  a value T that at least `m` of its lanes reach with their maximum and writes
 *                  every float4 group that holds an element >= T, with the index of the group's
 *                  first element, into the wavefront's own slots. Everything the wavefront does
 *                  not hand on is below T.
 *   k_final_cand   grid (rows). B = the largest T of the row's wavefronts: every element of the
 *                  row at or above B was handed on by its wavefront. If k of the handed-on
 *                  elements reach B (after the penalties, when those were left to this kernel),
 *                  the row's top k are among them (sampler.c:202-215 keeps the k largest of the
 *                  sorted row). They are penalised, cut to the k largest, ordered (logit
 *                  descending, index ascending: sampler.c:207 with a stable sort) and handed to the
 *                  common tail (softmax over the survivors, top-p, min-p, draw). A row that
 *                  cannot be certified this way -- leading logits crowded into one wavefront's
 *                  elements, runs of equal values, rows of -inf -- takes the thread-maxima path
 *                  (topk_from_tmax), which the scan also feeds, and from there the general one.
 *
 * `m` is chosen on the host so that a wavefront holding m of the row's leading logits is a
 * one-in-10^8 event for logits whose order is unrelated to the vocabulary order; it only
 * decides how often the slower path runs, never the token.
 *
 * The row-final kernel is bound by chains of dependent steps (a round trip to LDS, a reduction
 * over a wavefront, a barrier: 50 to 100 ns each with four wavefronts on a compute unit), not by
 * arithmetic. Hence: places in lists come from ballots and lane counts, not from atomics that
 * return a value; each wavefront keeps to its own share of the candidates for as long as it can;
 * the cut to the k largest and everything after it runs on one wavefront without barriers.
 */
#ifndef GEIST_SAMPLER_CANDS_H
#define GEIST_SAMPLER_CANDS_H

namespace gs {

constexpr uint32_t KEY_LOWEST_FINITE = 0x00800000u; /* f2key(-FLT_MAX) */
constexpr int      CAND_CUT_MAX      = CAND_K_MAX; /* entries the last wavefront orders */
static_assert(CAND_CUT_MAX == WAVE, "one entry per lane");

/* lanes of the wavefront for which `p` holds, as a mask (one comparison, no select) */
__device__ __forceinline__ uint64_t ballot64(bool p) { return __builtin_amdgcn_ballot_w64(p); }
/* set bits of `mask` below this lane */
__device__ __forceinline__ unsigned lanes_before(uint64_t mask) {
    return __builtin_amdgcn_mbcnt_hi((uint32_t) (mask >> 32),
                                     __builtin_amdgcn_mbcnt_lo((uint32_t) mask, 0u));
}
/* orders the LDS traffic of one wavefront: what its lanes wrote before is what they read after */
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ uint32_t hist_hash(int id) {
    return ((uint32_t) id * 0x9E3779B1u) >> 20; /* 12 bits: HT_SLOTS slots */
}

template <int NV>
__device__ __forceinline__ void cand_scan_chunk(const RowView &rv, float *__restrict__ tmax,
                                                const WaveCands &wc, int m, int row, int chunk,
                                                int tid) {
    const int lane = tid & (WAVE - 1);
    int       base, end;
    chunk_bounds<NV>(rv, chunk, base, end);
    float4 v[NV];
    load_raw<NV>(rv, rv.logits + (long) row * rv.ld, base, end, v, tid);
    float gm[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j)
        gm[j] = max3f(max3f(v[j].x, v[j].y, v[j].z), v[j].w, v[j].w);
    float tm = gm[0];
#pragma unroll
    for (int j = 1; j + 1 < NV; j += 2)
        tm = max3f(tm, gm[j], gm[j + 1]);
    if ((NV & 1) == 0)
        tm = max3f(tm, gm[NV - 1], gm[NV - 1]);
    if (base + 4 * tid >= end)
        tm = __builtin_nanf("");
    tmax[((long) row * rv.n_chunks + chunk) * TPB + tid] = tm;

    /* T: the largest value on the leading 16 key bits (sign, exponent, 7 bits of the fraction)
     * that m lanes reach. (The key is made opaque so that the NaN test inside f2key is not
     * repeated in every step.) */
    uint32_t key = f2key(tm);
    asm volatile("" : "+v"(key));
    uint32_t tau = 0u;
#pragma unroll
    for (int bit = 31; bit >= 16; --bit) {
        const uint32_t t = tau | (1u << bit);
        if (__popcll(ballot64(key >= t)) >= m)
            tau = t;
    }
    /* never below the lowest finite value: -inf (padding, forbidden tokens) is not handed on */
    tau           = tau < KEY_LOWEST_FINITE ? KEY_LOWEST_FINITE : tau;
    const float T = key2f(tau);
    /* which lanes hand group j on: one comparison per group; a lane's place among the
     * wavefront's groups is the number of groups before j plus its rank in group j's mask */
    uint64_t mk[NV];
    int      total = 0;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        mk[j] = ballot64(gm[j] >= T);
        total += __popcll(mk[j]);
    }
    const int  wvu   = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const long slot0 = ((long) row * (rv.n_chunks * NWAVES) + chunk * NWAVES + wvu);
    /* too many: nothing is handed on and the row cannot be certified */
    const bool fits = total <= CAND_GROUPS;
    if (lane == 0)
        wc.bound[slot0] = fits ? tau : 0xffffffffu;
    float4  *ov = wc.val + slot0 * CAND_SLOTS;
    int32_t *oi = wc.idx + slot0 * CAND_SLOTS;
    if (lane < CAND_GROUPS && (!fits || lane >= total))
        oi[lane] = -1; /* an unused slot */
    if (fits) {
        const int e0     = base + 4 * tid;
        unsigned  before = 0;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            if (gm[j] >= T) {
                const unsigned p = before + lanes_before(mk[j]);
                ov[p]            = v[j];
                oi[p]            = e0 + 4 * j * TPB;
            }
            before += (unsigned) __popcll(mk[j]);
        }
    }
}

template <int NV>
__global__ __launch_bounds__(TPB) void k_cand_scan(RowView rv, float *__restrict__ tmax,
                                                   WaveCands wc, int m) {
    int row, chunk;
    xcd_row_chunk(row, chunk);
    cand_scan_chunk<NV>(rv, tmax, wc, m, row, chunk, (int) threadIdx.x);
}

struct CandShared {
    uint32_t red_b[2];  /* largest bound among the row's first / second 64 scanning wavefronts */
    uint32_t mx;        /* largest key among the elements */
    int      n_real;    /* elements that still reach B after the penalties */
    int      n_cut;     /* entries listed for the final ordering */
    int      give_up;   /* the row cannot be served here */
};

constexpr int FC_THREADS = 1024;             /* threads of the final kernel */
constexpr int ARRIVE_STRIDE = ARRIVE_STRIDE_INTS; /* ints between the rows' arrival counters */
constexpr int FC_WAVES   = FC_THREADS / WAVE;
constexpr int FC_LIST    = 64;               /* elements at or above B one wavefront may hold */
constexpr int FC_STRIDE  = 2 * FC_LIST;      /* its list in LDS: FC_LIST entries, then one spare
                                              * slot per lane for the writes that do not count */

/* Layout of the final kernel's LDS arena while the candidate path runs (bytes). The thread-maxima
 * path, when a row falls back to it, reuses the arena from its start. */
constexpr int CA_EVAL = 0;                                   /* u32 [16][FC_STRIDE] bits, then keys */
constexpr int CA_EIDX = CA_EVAL + FC_WAVES * FC_STRIDE * 4;  /* u32 [16][FC_STRIDE] vocabulary ids  */
constexpr int CA_HKEY = CA_EIDX + FC_WAVES * FC_STRIDE * 4;  /* int [HT_SLOTS] the history table    */
constexpr int CA_HCNT = CA_HKEY + HT_SLOTS * 4;              /* u32 [HT_SLOTS / 2] occurrences      */
constexpr int CA_HIST = CA_HCNT + HT_SLOTS * 2;              /* u32 [256] key bins                  */
constexpr int CA_CUT  = CA_HIST + 256 * 4;                   /* u64 [2 * CAND_CUT_MAX]              */
constexpr int CA_END  = CA_CUT + 2 * CAND_CUT_MAX * 8;

/* Layout for the thread-maxima path and the general path behind it. */
template <int NV, bool PEN>
struct FallbackArena {
    static constexpr int BIG   = 0;                                   /* u8  [TMAX_LDS]        */
    static constexpr int MX    = BIG + TMAX_LDS;                      /* u32 [TPB]             */
    static constexpr int SELID = MX + TPB * 4;                        /* int [SEL_MAX]         */
    static constexpr int PCNT  = SELID + SEL_MAX * 4;                 /* u32 [SEL_MAX*4*NV]    */
    static constexpr int M     = PCNT + (PEN ? SEL_MAX * 4 * NV * 4 : 16); /* u64 [TPB]        */
    static constexpr int CNT16 = M + TPB * 8;                         /* u32 [NV*TPB*2]        */
    static constexpr int END   = CNT16 + (PEN ? NV * TPB * 2 * 4 : 16);
};

/* The rows the candidate path cannot certify: the thread-maxima path over the maxima the scan
 * stored, then the general one. Kept out of line: it is rare, and inlined it would be nine
 * tenths of the kernel's code. The first 256 threads of the workgroup call, after the others
 * have ended; returns the number of survivors in s_pack. */
template <int NV, bool PEN>
__device__ __forceinline__ int cand_fallback(const RowView *rvp, const FinalArgs *ap, int row,
                                          uint8_t *arena, uint64_t *s_pack, GeneralShared *gsp,
                                          int *s_n, int *s_n2) {
    using FA = FallbackArena<NV, PEN>;
    const RowView   &rv = *rvp;
    const FinalArgs &a  = *ap;
    int              k  = a.k;
    bool             general = true;
    if (rv.n_chunks <= 16)
        general = topk_from_tmax<NV, PEN, 16, false>(
            rv, a, row, arena + FA::BIG, reinterpret_cast<uint32_t *>(arena + FA::MX),
            reinterpret_cast<int *>(arena + FA::SELID),
            reinterpret_cast<uint32_t *>(arena + FA::PCNT),
            reinterpret_cast<uint64_t *>(arena + FA::M), s_pack, s_n, s_n2, k);
    else if (rv.n_chunks <= TMAX_LDS / TPB)
        general = topk_from_tmax<NV, PEN, TMAX_LDS / TPB, false>(
            rv, a, row, arena + FA::BIG, reinterpret_cast<uint32_t *>(arena + FA::MX),
            reinterpret_cast<int *>(arena + FA::SELID),
            reinterpret_cast<uint32_t *>(arena + FA::PCNT),
            reinterpret_cast<uint64_t *>(arena + FA::M), s_pack, s_n, s_n2, k);
    if (general) {
        __syncthreads();
        k = topk_row_general<NV, PEN, false>(rv, row, a.k, s_pack, TOPK_FAST_MAX,
                                             reinterpret_cast<uint32_t *>(arena + FA::CNT16), *gsp);
    }
    if (a.row_flag && threadIdx.x == 0)
        a.row_flag[row] = general ? 2 : 1; /* diagnostics: which path served the row */
    return k;
}

__device__ __forceinline__ double readlane_f64(double v, int lane) {
    const uint64_t u = (uint64_t) __double_as_longlong(v);
    return __longlong_as_double((long long) (((uint64_t) readlane_u32((uint32_t) (u >> 32), lane) << 32) |
                                             readlane_u32((uint32_t) u, lane)));
}

/* The common tail (finish_sorted_wave with one entry per lane) for n <= 64 survivors, written
 * for few instructions: lane i holds entry i, values travel by readlane, no LDS round trip
 * after the first read. Softmax over the survivors (sampler.c:219 via 68-85), normalisation
 * (sampler.c:251-253), nucleus (sampler.c:273-283), min-p prefix, draw (sampler.c:90-102).
 * Call with all 64 lanes of one wavefront. */
__device__ __forceinline__ int finish_sorted_lanes(int n, const uint64_t *spack, float inv_t,
                                                   float top_p, float min_p, float u,
                                                   const uint64_t *tab) {
    const int      lane  = threadIdx.x & (WAVE - 1);
    const bool     use_p = top_p > 0.0f && top_p < 1.0f;
    const bool     use_m = min_p > 0.0f;
    const bool     in    = lane < n;
    const uint64_t mine  = spack[in ? lane : 0];
    const float    l     = key2f(best_key(mine));
    const float    l0    = __uint_as_float(readlane_u32(__float_as_uint(l), 0));
    float          w     = in ? geist_expf_glibc_le0(softmax_arg(l, l0, inv_t), tab) : 0.0f;
    double         c     = wave_scan_f64_dpp((double) w);
    if (use_p || use_m) {
        const double sum = readlane_f64(c, WAVE - 1);
        w                = in ? (float) ((double) w / sum) : 0.0f;
        c                = wave_scan_f64_dpp((double) w);
    }
    int keep = n;
    if (use_p) {
        const uint64_t mk = ballot64(in && c >= (double) top_p);
        if (mk)
            keep = __ffsll((long long) mk); /* first crossing entry, inclusive */
    }
    if (use_m) {
        const float floor_w = __fmul_rn(min_p, __uint_as_float(readlane_u32(__float_as_uint(w), 0)));
        int         m       = __popcll(ballot64(in && w >= floor_w));
        m                   = m < 1 ? 1 : m;
        keep                = m < keep ? m : keep;
    }
    keep                  = keep < 1 ? 1 : keep;
    const double   target = (double) u * readlane_f64(c, keep - 1);
    const uint64_t hk     = ballot64(lane < keep && target < c);
    const int      at     = hk ? __ffsll((long long) hk) - 1 : keep - 1;
    return (int) (0xffffffffu - readlane_u32((uint32_t) mine, at));
}

static_assert(CAND_GROUPS == 32 && CAND_SLOTS == 32, "the slot-to-thread maps below");

/* One workgroup of 1024 threads per row, so that every wavefront has little to do and a SIMD's
 * four wavefronts cover each other's waits. WIDE = false: up to 64 scanning wavefronts per row;
 * thread t reads slots (t & 15) and 16 + (t & 15) of scanning wavefront t >> 4. WIDE = true: up
 * to 128; slots (t & 7) + 8 r, r < 4, of wavefront t >> 3. */
template <int NV, bool PEN, bool WIDE>
__device__ __forceinline__ void final_cand_row(const RowView &rv, const FinalArgs &a,
                                               const WaveCands &wc, int row) {
    constexpr int ROUNDS = WIDE ? 4 : 2;
    constexpr int ARENA = CA_END > FallbackArena<NV, PEN>::END ? CA_END : FallbackArena<NV, PEN>::END;
    __shared__ __align__(16) uint8_t s_arena[ARENA];
    __shared__ uint64_t      s_tab[32];
    __shared__ uint64_t      s_pack[TOPK_FAST_MAX];
    __shared__ GeneralShared s_gs;
    __shared__ CandShared    s_c;
    __shared__ int           s_n, s_n2;
    const int tid = threadIdx.x, lane = tid & (WAVE - 1);
    const int wv  = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int W   = rv.n_chunks * NWAVES; /* wavefronts that scanned the row */
    uint32_t *e_val = reinterpret_cast<uint32_t *>(s_arena + CA_EVAL) + wv * FC_STRIDE;
    uint32_t *e_idx = reinterpret_cast<uint32_t *>(s_arena + CA_EIDX) + wv * FC_STRIDE;
    int      *hkey  = reinterpret_cast<int *>(s_arena + CA_HKEY);
    uint32_t *hcnt  = reinterpret_cast<uint32_t *>(s_arena + CA_HCNT);
    uint32_t *hist  = reinterpret_cast<uint32_t *>(s_arena + CA_HIST);
    uint64_t *s_cut = reinterpret_cast<uint64_t *>(s_arena + CA_CUT);
    /* every load this kernel needs from memory is issued here, before anything is waited for */
    float4 gv[ROUNDS];
    int    gi[ROUNDS];
    {
        const int      ws  = WIDE ? tid >> 3 : tid >> 4;
        const int      p0  = WIDE ? tid & 7 : tid & 15;
        const unsigned at0 = ((unsigned) row * (unsigned) W + (unsigned) ws) * CAND_SLOTS + (unsigned) p0;
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r) {
            const int p = p0 + (WIDE ? 8 : 16) * r;
            gi[r]       = -1;
            gv[r]       = make_float4(0.f, 0.f, 0.f, 0.f);
            if (ws < W && p < CAND_GROUPS) {
                gv[r] = wc.val[at0 + (WIDE ? 8 : 16) * r];
                gi[r] = wc.idx[at0 + (WIDE ? 8 : 16) * r];
            }
        }
    }
    uint32_t bk = tid < W ? wc.bound[row * W + tid] : 0u;
    /* the row's history: the first two ids of each thread are asked for here (2048 ids: all of
     * most histories), the rest when the history is looked up */
    int            hid0 = -1, hid1 = -1, hlen = 0;
    const int32_t *hrow = nullptr;
    if (PEN) {
        hlen = rv.hist_len[row];
        hlen = hlen > rv.hist_ld ? (int) rv.hist_ld : hlen;
        hrow = rv.hist + (long) row * rv.hist_ld;
        if (tid < hlen)
            hid0 = hrow[tid];
        if (tid + FC_THREADS < hlen)
            hid1 = hrow[tid + FC_THREADS];
    }
    const float u_row = a.uniforms[row];
    if (tid < 32)
        s_tab[tid] = g_expf_tab[tid];
    if (tid < 256)
        hist[tid] = 0u;
    if (tid == 0) {
        s_c.mx      = 0u;
        s_c.n_real  = 0;
        s_c.n_cut   = 0;
        s_c.give_up = 0;
    }
    if (PEN) { /* the history table starts empty */
        static_assert(HT_SLOTS == 4 * FC_THREADS, "one 16-byte piece of each array per thread");
        reinterpret_cast<uint4 *>(hkey)[tid] = make_uint4(~0u, ~0u, ~0u, ~0u);
        if (tid < HT_SLOTS / 8)
            reinterpret_cast<uint4 *>(hcnt)[tid] = make_uint4(0u, 0u, 0u, 0u);
    }
    /* B: the largest bound of the row's wavefronts (they sit in the first W <= 128 threads) */
    if (wv < 2) {
        bk = wave_max_u32(bk);
        if (lane == 0)
            s_c.red_b[wv] = bk;
    }
    __syncthreads();
    bk = s_c.red_b[0] > s_c.red_b[1] ? s_c.red_b[0] : s_c.red_b[1];
    /* 0xffffffff: a wavefront of the scan had more groups than slots */
    bool           give_up = bk == 0xffffffffu;
    const uint32_t lo      = bk < KEY_LOWEST_FINITE ? KEY_LOWEST_FINITE : bk;
    const float    B       = key2f(lo);
    /* With penalties the table in LDS is of the CANDIDATES (a few hundred ids, each once), and
     * the row's history is looked up in it: an id of the history that is no candidate -- nearly
     * all of them -- costs one LDS read, and only hits count, with an atomic add. (A table of
     * the history's 2048 ids took two to three returning atomics per id, and the most frequent
     * ids' additions queued behind one another.) */
    const bool have0 = PEN && (unsigned) hid0 < (unsigned) rv.n_vocab;
    const bool have1 = PEN && (unsigned) hid1 < (unsigned) rv.n_vocab;
    /* this wavefront's elements at or above B, into its list in LDS. A lane's place is the
     * number of kept elements before it; what is not kept is written to the lane's spare slot,
     * so that no branch is needed. */
    unsigned n_e = 0;
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const float    xc   = f4_get(gv[r], c);
            const bool     keep = gi[r] >= 0 && xc >= B;
            const uint64_t mk   = ballot64(keep);
            const unsigned p    = n_e + lanes_before(mk);
            const bool     put  = keep && p < (unsigned) FC_LIST;
            const unsigned at   = put ? p : (unsigned) (FC_LIST + lane);
            e_val[at]           = (PEN || a.cap_after) ? __float_as_uint(xc) : f2key(xc);
            e_idx[at]           = (uint32_t) (gi[r] + c);
            n_e += (unsigned) __popcll(mk);
        }
    }
    give_up = give_up || n_e > (unsigned) FC_LIST;
    /* one element per lane from here on */
    wave_lds_sync();
    uint32_t my_slot = 0u;
    if (PEN) {
        /* every listed element claims a slot (ids of a row are distinct: a claim never meets
         * its own id; at most 16 x 64 elements for 4096 slots) */
        if (lane < (int) (n_e < (unsigned) FC_LIST ? n_e : (unsigned) FC_LIST)) {
            const int id = (int) e_idx[lane];
            my_slot      = hist_hash(id);
#pragma unroll 1
            for (int pr = 0; pr < HT_SLOTS && atomicCAS(&hkey[my_slot], -1, id) != -1; ++pr)
                my_slot = (my_slot + 1u) & (HT_SLOTS - 1);
        }
        __syncthreads();
        /* the history: a hit adds one to the element's counter (16-bit counters, two a word: a
         * history holds fewer than 65536 ids) */
        auto look_up = [&](int id) {
            uint32_t h = hist_hash(id);
            int      k = hkey[h];
#pragma unroll 1
            for (int pr = 0; pr < HT_SLOTS && k != id && k != -1; ++pr) {
                h = (h + 1u) & (HT_SLOTS - 1);
                k = hkey[h];
            }
            if (k == id)
                atomicAdd(&hcnt[h >> 1], 1u << (16 * (h & 1u)));
        };
        if (have0)
            look_up(hid0);
        if (have1)
            look_up(hid1);
#pragma unroll 1
        for (int i = tid + 2 * FC_THREADS; i < hlen; i += FC_THREADS) {
            const int id = hrow[i];
            if ((unsigned) id < (unsigned) rv.n_vocab)
                look_up(id);
        }
        __syncthreads();
    }
    /* With penalties: how often the row's history names the element is read from its slot; an
     * element that no longer reaches B gets key 0. */
    uint32_t my_key = 0u;
    /* With the soft-cap left to this kernel (FinalArgs::cap_after) an entry counts when its
     * capped value lies strictly above the capped bound: those are certain to be all there are. */
    const float Bc = a.cap_after ? softcap1(B, rv.softcap) : B;
    if (!give_up && lane < (int) n_e) {
        my_key = e_val[lane];
        if (PEN || a.cap_after) {
            float x = __uint_as_float(my_key);
            if (PEN) {
                const uint32_t times = (hcnt[my_slot >> 1] >> (16 * (my_slot & 1u))) & 0xffffu;
                if (times)
                    x = penalise(x, times, rv.rep, rv.inv_rep, rv.freq, rv.pres);
            }
            if (a.cap_after) {
                my_key = 0u;
                if (x >= B) {
                    const float xc = softcap1(x, rv.softcap);
                    my_key         = xc > Bc ? f2key(xc) : 0u;
                }
            } else {
                my_key = x >= B ? f2key(x) : 0u;
            }
        }
    }
    {
        const int      real = __popcll(ballot64(my_key != 0u));
        const uint32_t mxk  = wave_max_u32(my_key);
        if (lane == 0 && real) {
            atomicMax(&s_c.mx, mxk);
            atomicAdd(&s_c.n_real, real);
        }
    }
    if (give_up)
        s_c.give_up = 1;
    __syncthreads();
    give_up = s_c.give_up != 0;
    /* The k largest. The keys lie in [lo_k, mx]; 256 bins over that range, counted by all
     * wavefronts, then every wavefront finds the bin in which the count from above reaches k.
     * The entries from that bin upwards are listed; should they be more than CAND_CUT_MAX the
     * bin is split again. */
    const int n_real = s_c.n_real;
    give_up = give_up || n_real < a.k; /* fewer than k at or above B: B certifies nothing */
    /* (keys of capped values lie above the capped bound's, which is below the raw bound's) */
    const uint32_t lo_k = a.cap_after ? f2key(Bc) : lo;
    uint32_t cut = lo_k; /* entries with key >= cut are listed */
    if (!give_up && n_real > CAND_CUT_MAX) {
        uint32_t base_k = lo_k, top_k = s_c.mx; /* the range being split, inclusive */
        int      need        = a.k;       /* entries wanted from this range: its `need` largest */
        int      above_total = 0;         /* entries above the range: all of them are wanted */
        int      listed      = n_real;    /* entries at or above the cut */
#pragma unroll 1
        for (int pass = 0; pass < 4 && listed > CAND_CUT_MAX; ++pass) {
            const uint32_t range = top_k - base_k;
            const int      sh    = range < 256u ? 0 : 24 - __clz((int) range);
            if (pass) {
                __syncthreads();
                if (tid < 256)
                    hist[tid] = 0u;
                __syncthreads();
            }
            if (my_key >= base_k && my_key <= top_k)
                atomicAdd(&hist[(my_key - base_k) >> sh], 1u);
            __syncthreads();
            /* lane l looks at bins 252 - 4 l .. 255 - 4 l; the count runs from the top bin down */
            const uint4    hb      = *reinterpret_cast<const uint4 *>(&hist[252 - 4 * lane]);
            const int      s4      = (int) (hb.x + hb.y + hb.z + hb.w);
            const int      inc     = wave_scan_i32_dpp(s4);
            const uint64_t crossed = ballot64(inc >= need);
            /* (some lane crosses: the range holds at least `need` entries) */
            const int L   = crossed ? __ffsll((long long) crossed) - 1 : WAVE - 1;
            const int run = inc - s4;
            /* in lane L: the first bin from the top at which the count reaches `need` */
            int off = 0, got = inc, here = (int) hb.x;
            if (run + (int) hb.w >= need)
                off = 3, got = run + (int) hb.w, here = (int) hb.w;
            else if (run + (int) (hb.w + hb.z) >= need)
                off = 2, got = run + (int) (hb.w + hb.z), here = (int) hb.z;
            else if (run + (int) (hb.w + hb.z + hb.y) >= need)
                off = 1, got = run + (int) (hb.w + hb.z + hb.y), here = (int) hb.y;
            const int bin = 252 - 4 * L + (int) readlane_u32((uint32_t) off, L);
            got           = (int) readlane_u32((uint32_t) got, L);
            const int above = got - (int) readlane_u32((uint32_t) here, L);
            const uint32_t bin_lo = base_k + ((uint32_t) bin << sh);
            cut                   = bin_lo;
            listed                = above_total + got;
            if (listed > CAND_CUT_MAX) {
                if (sh == 0)
                    break; /* one key value fills the bin: a run of equal values */
                /* everything above the bin is wanted; the bin itself is split again */
                above_total += above;
                need -= above;
                const uint32_t bin_hi = bin_lo + ((1u << sh) - 1u);
                base_k                = bin_lo;
                top_k                 = bin_hi < top_k ? bin_hi : top_k;
            }
        }
        give_up = give_up || listed > CAND_CUT_MAX; /* runs of equal values */
    }
    if (!give_up) {
        /* the entries that reach the cut: each wavefront lists its own, after asking for places
         * (cut > 0: a dropped entry's key 0 never passes) */
        const bool     keep = my_key >= cut;
        const uint64_t mk   = ballot64(keep);
        int            base_p = 0;
        if (lane == 0 && mk)
            base_p = atomicAdd(&s_c.n_cut, (int) __popcll(mk));
        const unsigned p = (unsigned) __builtin_amdgcn_readfirstlane(base_p) + lanes_before(mk);
        if (keep && p < 2u * CAND_CUT_MAX)
            s_cut[p] = pack_best(my_key, e_idx[lane]);
    } else {
        s_c.give_up = 1;
    }
    __syncthreads();
    give_up = s_c.give_up != 0 || s_c.n_cut > CAND_CUT_MAX;
    if (!give_up) {
        /* order by counting (logit descending, index ascending): entry i is compared with the
         * others by sixteen neighbouring lanes, whose counts a row of DPP shifts adds up */
        const int      n_c = s_c.n_cut;
        const int      i = tid >> 4, part = tid & 15;
        const uint64_t me   = i < n_c ? s_cut[i] : 0ull;
        int            rank = 0;
#pragma unroll
        for (int q = 0; q < CAND_CUT_MAX / 16; ++q) {
            const int j = part + 16 * q;
            rank += j < n_c && s_cut[j] > me;
        }
        rank += __builtin_amdgcn_update_dpp(0, rank, 0x111, 0xf, 0xf, false); /* row_shr:1 */
        rank += __builtin_amdgcn_update_dpp(0, rank, 0x112, 0xf, 0xf, false); /* row_shr:2 */
        rank += __builtin_amdgcn_update_dpp(0, rank, 0x114, 0xf, 0xf, false); /* row_shr:4 */
        rank += __builtin_amdgcn_update_dpp(0, rank, 0x118, 0xf, 0xf, false); /* row_shr:8 */
        if (i < n_c && part == 15 && rank < a.k)
            s_pack[rank] = me;
    }
    __syncthreads();
    /* all but the first wavefront are done, or all but the first four when the row falls back
     * (the slower paths are written for 256 threads) */
    if (tid >= (give_up ? TPB : WAVE))
        return;
    int k = a.k;
    if (give_up)
        k = cand_fallback<NV, PEN>(&rv, &a, row, s_arena, s_pack, &s_gs, &s_n, &s_n2);
    else if (a.row_flag && tid == 0)
        a.row_flag[row] = 0;
    if (tid < WAVE) {
        /* (k <= CAND_K_MAX = 64 on this path) */
        const int tok = finish_sorted_lanes(k, s_pack, a.inv_t, a.top_p, a.min_p, u_row, s_tab);
        if (tid == 0)
            a.out[row] = tok;
    }
}

template <int NV, bool PEN, bool WIDE>
__global__ __launch_bounds__(FC_THREADS) void k_final_cand(RowView rv, FinalArgs a, WaveCands wc) {
    final_cand_row<NV, PEN, WIDE>(rv, a, wc, (int) blockIdx.x);
}

} // namespace gs
#endif
