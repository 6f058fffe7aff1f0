/*
 * sampler_kernels.hip -- the HIP kernels of the token-sampling path (gfx950).
 *
 * Kernel map (reference lines the arithmetic follows are cited at each kernel):
 *   k_chunk_best     per-(row, chunk) maximum with lowest-index tie-break     sampler.c:52-62, 70-75
 *   k_chunk_expsum   per-(row, chunk) sum of expf((l - max) * inv_t)          sampler.c:77-83
 *   k_topk_scan      per-(row, chunk) candidates that can be in the top k     sampler.c:202-207
 *   k_row_final      per-row combine: argmax / index-order CDF draw / top-k
 *                    select, sorted softmax, top-p, min-p, draw               sampler.c:90-102, 209-222, 272-299
 *   k_write_probs    normalised probabilities of a row                        sampler.c:246-253
 *   k_penalties      in-place penalties                                       (no reference counterpart)
 *   k_rng_units      xorshift64* uniforms                                     sampler.c:35-48
 *
 * All streaming kernels use a (n_chunks, rows) grid of 256-thread workgroups and read each
 * logit exactly once per kernel; the logits are never written (k_penalties excepted).
 */
#include "sampler_kernels.h"

#include "sampler_device.h"

#include <type_traits>

namespace gs {

__device__ const uint64_t g_expf_tab[32] = GEIST_EXPF_TABLE_INIT;

/* Phase timestamps for kernel tuning; compiled in only by the tuning probe. */
#ifdef GS_PHASES
__device__ long long g_phase[16384 * 8];
#define GS_MARK(i)                                                                             \
    do {                                                                                       \
        if (threadIdx.x == 0)                                                                  \
            g_phase[((long) blockIdx.y * gridDim.x + blockIdx.x) * 8 + (i)] = wall_clock64();   \
    } while (0)
#else
#define GS_MARK(i) ((void) 0)
#endif

/* number of leading key bits the per-chunk threshold search resolves */
constexpr int THR_BITS = 16;

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
template <int NV, bool PEN>
__device__ __forceinline__ void fetch_chunk(const RowView &rv, int row, int base, int end,
                                            uint32_t *cnt16, float4 (&v)[NV]) {
    const float *rowp = rv.logits + (long) row * rv.ld;
    if (PEN) {
        history_clear<NV * TPB * 4>(cnt16);
        load_raw<NV>(rv, rowp, base, end, v);
        history_count(rv, row, base, end, cnt16);
        apply_transform<NV>(rv, cnt16, v);
    } else {
        load_raw<NV>(rv, rowp, base, end, v);
        apply_transform<NV>(rv, nullptr, v);
    }
}

/* ============================================================================================
 * k_chunk_best: the maximum of each chunk and where it first occurs.
 * ========================================================================================== */
template <int NV, bool PEN>
__global__ __launch_bounds__(TPB) void k_chunk_best(RowView rv, uint64_t *__restrict__ chunk_best) {
    __shared__ __align__(16) uint32_t s_cnt16[PEN ? NV * TPB * 2 : 1];
    __shared__ uint64_t s_red[NWAVES];
    const int           row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
    int                 base, end;
    chunk_bounds<NV>(rv, chunk, base, end);
    float4 v[NV];
    fetch_chunk<NV, PEN>(rv, row, base, end, s_cnt16, v);

    uint64_t best = 0;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int e = base + 4 * (j * TPB + tid);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            if (e + c < end) {
                const uint64_t p = pack_best(f2key(f4_get(v[j], c)), (uint32_t) (e + c));
                best             = p > best ? p : best;
            }
        }
    }
    best = block_max_u64(best, s_red);
    if (tid == 0)
        chunk_best[(long) row * rv.n_chunks + chunk] = best;
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
 * k_chunk_expsum: sum over the chunk of p_i = expf((l_i - max) * inv_t), in double.
 * Optionally records p at one token of the row (spec verification needs p(x_j)).
 * ========================================================================================== */
template <int NV, bool PEN>
__global__ __launch_bounds__(TPB) void k_chunk_expsum(RowView rv, float inv_t,
                                                      const uint64_t *__restrict__ chunk_best,
                                                      double *__restrict__ chunk_sum,
                                                      const int32_t *__restrict__ probe_token,
                                                      float *__restrict__ probe_p) {
    __shared__ __align__(16) uint32_t s_cnt16[PEN ? NV * TPB * 2 : 1];
    __shared__ uint64_t s_red[NWAVES];
    __shared__ double   s_sum[NWAVES];
    __shared__ uint64_t s_tab[32];
    const int           row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
    if (tid < 32)
        s_tab[tid] = g_expf_tab[tid];
    int base, end;
    chunk_bounds<NV>(rv, chunk, base, end);
    float4 v[NV];
    fetch_chunk<NV, PEN>(rv, row, base, end, s_cnt16, v);
    const float mx = key2f(best_key(row_best_from_chunks(chunk_best, row, rv.n_chunks, s_red)));

    const int tok = probe_token ? probe_token[row] : -1;
    double    acc = 0.0;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int e = base + 4 * (j * TPB + tid);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            if (e + c < end) {
                const float p = geist_expf_glibc(softmax_arg(f4_get(v[j], c), mx, inv_t), s_tab);
                acc += (double) p;
                if (e + c == tok)
                    probe_p[row] = p;
            }
        }
    }
    acc = block_sum_f64(acc, s_sum);
    if (tid == 0)
        chunk_sum[(long) row * rv.n_chunks + chunk] = acc;
}

/* ============================================================================================
 * k_topk_scan: every element of the chunk that can belong to the row's top k.
 *
 * The workgroup's 256 per-thread maxima are folded into G = 64, 128 or 256 group maxima; the
 * k-th largest of them is a lower bound of the chunk's k-th largest element, so every element
 * at or above it is kept (about -G ln(1 - k/G) of them). The bound is found on the leading
 * THR_BITS of the order-preserving key by a bitwise search with wavefront ballots. Comparisons
 * on the elements themselves stay in fp32: max ignores NaN and `!(x < bound)` keeps it, which
 * is what the key order prescribes. A chunk that yields more than `cap` candidates reports its
 * true count and the row takes the general path.
 * ========================================================================================== */
template <int VPL>
__device__ __forceinline__ uint32_t kth_group_max(uint32_t q0, uint32_t q1, uint32_t q2,
                                                  uint32_t q3, int kk) {
    uint32_t tau = 0;
#pragma unroll
    for (int bit = 31; bit >= 32 - THR_BITS; --bit) {
        const uint32_t t   = tau | (1u << bit);
        int            cnt = __popcll(__ballot(q0 >= t));
        if (VPL >= 2)
            cnt += __popcll(__ballot(q1 >= t));
        if (VPL >= 4)
            cnt += __popcll(__ballot(q2 >= t)) + __popcll(__ballot(q3 >= t));
        if (cnt >= kk)
            tau = t;
    }
    return tau;
}

template <int NV, bool PEN>
__global__ __launch_bounds__(TPB) void k_topk_scan(RowView rv, int k, int cap,
                                                   uint64_t *__restrict__ cand_pack,
                                                   int32_t *__restrict__ cand_cnt) {
    __shared__ __align__(16) uint32_t s_cnt16[PEN ? NV * TPB * 2 : 1];
    __shared__ float    s_tmax[TPB];
    __shared__ uint64_t s_cand[TOPK_CAND_CAP];
    __shared__ int      s_n;
    const int           row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
    const int           lane = tid & (WAVE - 1);
    int                 base, end;
    chunk_bounds<NV>(rv, chunk, base, end);
    GS_MARK(0);
    float4 v[NV];
    fetch_chunk<NV, PEN>(rv, row, base, end, s_cnt16, v);

    float tm = -__builtin_inff();
#pragma unroll
    for (int j = 0; j < NV; ++j)
        tm = max3f(tm, max3f(v[j].x, v[j].y, v[j].z), v[j].w);
    s_tmax[tid] = tm;
    if (tid == 0)
        s_n = 0;
    GS_MARK(1);
    __syncthreads();
    GS_MARK(2);

    const float g0 = s_tmax[lane], g1 = s_tmax[lane + 64], g2 = s_tmax[lane + 128],
                g3 = s_tmax[lane + 192];
    uint32_t tau;
    if (k <= 24) {
        tau = kth_group_max<1>(f2key(max3f(max3f(g0, g1, g2), g3, g3)), 0, 0, 0, k);
    } else if (k <= 64) {
        tau = kth_group_max<2>(f2key(max3f(g0, g2, g2)), f2key(max3f(g1, g3, g3)), 0, 0, k);
    } else {
        tau = kth_group_max<4>(f2key(g0), f2key(g1), f2key(g2), f2key(g3), k < TPB ? k : TPB);
    }
    const float bound = key2f(tau); /* tau == 0 maps to NaN: nothing is below it */
    GS_MARK(3);

    /* Padding holds -inf, so with a finite bound no index test is needed on the hot path. */
    const bool check_idx = !(bound > -__builtin_inff());
    if (!(tm < bound)) {
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const float m4 = f4_max(v[j]);
            if (!(m4 < bound) || check_idx) {
                const int e = base + 4 * (j * TPB + tid);
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const float x = f4_get(v[j], c);
                    if (!(x < bound) && (!check_idx || e + c < end)) {
                        const int pos = atomicAdd(&s_n, 1);
                        if (pos < cap)
                            s_cand[pos] = pack_best(f2key(x), (uint32_t) (e + c));
                    }
                }
            }
        }
    }
    GS_MARK(4);
    __syncthreads();
    const int  n = s_n;
    const long o = (long) row * rv.n_chunks + chunk;
    if (tid == 0)
        cand_cnt[o] = n;
    const int m = n < cap ? n : cap;
    for (int i = tid; i < m; i += TPB)
        cand_pack[o * cap + i] = s_cand[i];
    GS_MARK(5);
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
#define GS_P(i) geist_expf_glibc(softmax_arg(key2f(best_key(spack[i])), l0, inv_t), fs.tab)

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
        if (use_p && first_p != 0x7fffffff)
            atomicMin(&fs.n_p, first_p);
        if (use_m && cnt_m)
            atomicAdd(&fs.n_m, cnt_m);
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
        double run = off;
        for (int i = lo; i < hi && i < keep; ++i) {
            run += (double) GS_W(i);
            if (target < run) {
                atomicMin(&fs.pick, i);
                break;
            }
        }
    }
    __syncthreads();
#undef GS_P
#undef GS_W
    const int at = fs.pick == 0x7fffffff ? keep - 1 : fs.pick;
    return (int) best_idx(spack[at]);
}

/* finish_sorted for n <= 128 survivors on ONE wavefront (call with all 64 lanes of a single
 * wave): lane l owns entries 2l and 2l+1, the prefix sums are wavefront scans, no barrier.
 * `tab` is the expf table in LDS. */
__device__ int finish_sorted_wave(int n, const uint64_t *spack, float inv_t, float top_p,
                                  float min_p, float u, const uint64_t *tab) {
    const int  lane  = threadIdx.x & (WAVE - 1);
    const bool use_p = top_p > 0.0f && top_p < 1.0f;
    const bool use_m = min_p > 0.0f;
    const bool norm  = use_p || use_m;
    const int  i0 = 2 * lane, i1 = 2 * lane + 1;
    const float l0 = key2f(best_key(spack[0]));
    float w0 = i0 < n ? geist_expf_glibc(softmax_arg(key2f(best_key(spack[i0])), l0, inv_t), tab)
                      : 0.0f;
    float w1 = i1 < n ? geist_expf_glibc(softmax_arg(key2f(best_key(spack[i1])), l0, inv_t), tab)
                      : 0.0f;
    double part = (double) w0 + (double) w1;
    double incl = wave_scan_f64(part);
    if (norm) {
        const double sum = __shfl(incl, WAVE - 1, WAVE);
        w0   = i0 < n ? (float) ((double) w0 / sum) : 0.0f;
        w1   = i1 < n ? (float) ((double) w1 / sum) : 0.0f;
        part = (double) w0 + (double) w1;
        incl = wave_scan_f64(part);
    }
    const double c0 = (incl - part) + (double) w0; /* inclusive prefix at entry i0 */
    const double c1 = c0 + (double) w1;            /* ... at entry i1 */
    int keep = n;
    if (use_p) {
        const uint64_t m0 = __ballot(i0 < n && c0 >= (double) top_p);
        const uint64_t m1 = __ballot(i1 < n && c1 >= (double) top_p);
        int first = n - 1;
        if (m0) first = 2 * (__ffsll((long long) m0) - 1);
        if (m1) {
            const int f1 = 2 * (__ffsll((long long) m1) - 1) + 1;
            first = (m0 && first < f1) ? first : f1;
        }
        keep = (m0 | m1) ? first + 1 : n;
    }
    if (use_m) {
        const float floor_w = __fmul_rn(min_p, __shfl(w0, 0, WAVE));
        int m = __popcll(__ballot(i0 < n && w0 >= floor_w)) +
                __popcll(__ballot(i1 < n && w1 >= floor_w));
        if (m < 1) m = 1;
        keep = m < keep ? m : keep;
    }
    if (keep < 1) keep = 1;
    const double   at_keep = ((keep - 1) & 1) ? c1 : c0;
    const double   mass    = __shfl(at_keep, (keep - 1) >> 1, WAVE);
    const double   target  = (double) u * mass;
    const uint64_t h0 = __ballot(i0 < keep && target < c0);
    const uint64_t h1 = __ballot(i1 < keep && target < c1);
    int at = keep - 1;
    if (h0 | h1) {
        const int f0 = h0 ? 2 * (__ffsll((long long) h0) - 1) : 0x7fffffff;
        const int f1 = h1 ? 2 * (__ffsll((long long) h1) - 1) + 1 : 0x7fffffff;
        at = f0 < f1 ? f0 : f1;
    }
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

template <int NV, bool PEN>
__device__ int topk_row_general(const RowView &rv, int row, int k_want, uint64_t *spack,
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
            fetch_chunk<NV, PEN>(rv, row, base, end, cnt16, v);
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
        fetch_chunk<NV, PEN>(rv, row, base, end, cnt16, v);
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

/* ============================================================================================
 * k_row_final: one workgroup per row.
 * ========================================================================================== */
struct FinalArgs {
    int   mode; /* FINAL_ARGMAX, FINAL_TEMPERATURE, FINAL_TOPK */
    int   k;
    int   cap;
    float inv_t;
    float top_p;
    float min_p;
    const float   *uniforms;
    const uint64_t *chunk_best;
    const double   *chunk_sum;
    const uint64_t *cand_pack;
    const int32_t  *cand_cnt;
    int32_t        *out;
};

template <int NV, bool PEN>
__global__ __launch_bounds__(TPB) void k_row_final(RowView rv, FinalArgs a) {
    __shared__ uint64_t      s_red[NWAVES];
    __shared__ FinishShared  s_fs;
    __shared__ GeneralShared s_gs;
    __shared__ uint64_t      s_cpack[FINAL_CAND_MAX];
    __shared__ uint64_t      s_m[TPB];
    __shared__ uint64_t      s_pack[TOPK_FAST_MAX];
    __shared__ double        s_csum[MAX_CHUNKS];
    __shared__ uint32_t      s_kmin, s_kmax;
    __shared__ __align__(16) uint32_t s_cnt16[PEN ? NV * TPB * 2 : 1];
    __shared__ int           s_off[MAX_CHUNKS + 1];
    __shared__ int           s_n, s_nt, s_chunk;
    __shared__ double        s_before;

    const int row = blockIdx.x, tid = threadIdx.x;
    const int C = rv.n_chunks;

    if (a.mode == FINAL_ARGMAX) {
        /* sampler.c:52-62 */
        const uint64_t b = row_best_from_chunks(a.chunk_best, row, C, s_red);
        if (tid == 0) {
            const float first = rv.logits[(long) row * rv.ld];
            /* a NaN at index 0 is never displaced by the strict '>' of the reference; after the
             * transforms it stays NaN, so the raw value decides */
            a.out[row] = (first != first) ? 0 : (int32_t) best_idx(b);
        }
        return;
    }

    if (a.mode == FINAL_TEMPERATURE) {
        /* sampler.c:90-102 over all n in index order: locate the chunk from the per-chunk sums,
         * then scan that chunk. */
        if (tid < C)
            s_csum[tid] = a.chunk_sum[(long) row * C + tid];
        if (tid < 32)
            s_fs.tab[tid] = g_expf_tab[tid];
        const float u_row = a.uniforms[row];
        __syncthreads();
        if (tid == 0) {
            double tot = 0.0;
            for (int c = 0; c < C; ++c)
                tot += s_csum[c];
            const double target = (double) u_row * tot;
            double       run    = 0.0;
            int          at     = C - 1;
            for (int c = 0; c < C; ++c) {
                const double nxt = run + s_csum[c];
                if (target < nxt || c == C - 1) {
                    at = c;
                    break;
                }
                run = nxt;
            }
            s_chunk   = at;
            s_before  = run;
            s_fs.mass = target;
        }
        const float mx = key2f(best_key(row_best_from_chunks(a.chunk_best, row, C, s_red)));
        /* (row_best_from_chunks ends with a barrier: s_chunk, s_before, tab are visible) */
        const int chunk = s_chunk;
        int       base, end;
        chunk_bounds<NV>(rv, chunk, base, end);
        float4 v[NV];
        fetch_chunk<NV, PEN>(rv, row, base, end, s_cnt16, v);
        /* index order inside the chunk is (j, thread, component): scan one j-slab at a time */
        double       carry  = s_before;
        const double target = s_fs.mass;
        if (tid == 0)
            s_fs.pick = 0x7fffffff;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int e = base + 4 * (j * TPB + tid);
            float     p[4];
            double    part = 0.0;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                p[c] = (e + c < end)
                           ? geist_expf_glibc(softmax_arg(f4_get(v[j], c), mx, a.inv_t), s_fs.tab)
                           : 0.0f;
                part += (double) p[c];
            }
            double       slab;
            const double incl = block_scan_f64(part, s_fs.scan, &slab);
            double       run  = carry + (incl - part);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                run += (double) p[c];
                if (e + c < end && target < run) {
                    atomicMin(&s_fs.pick, e + c);
                    break;
                }
            }
            carry += slab;
        }
        __syncthreads();
        if (tid == 0)
            a.out[row] = s_fs.pick == 0x7fffffff ? end - 1 : s_fs.pick;
        return;
    }

    /* ---- FINAL_TOPK: merge the per-chunk candidates ---------------------------------------- */
    if (tid < 32)
        s_fs.tab[tid] = g_expf_tab[tid];
    const float u_row = a.uniforms[row];
    int         n_c   = 0;
    bool        over  = false;
    if (tid < C) {
        const int raw = a.cand_cnt[(long) row * C + tid];
        over          = raw > a.cap;
        n_c           = over ? a.cap : raw;
    }
    int       N;
    const int incl = block_scan_i32(n_c, s_gs.scan, &N);
    if (tid < C)
        s_off[tid] = incl - n_c;
    if (tid == 0) {
        s_off[C] = N;
        s_n      = 0;
        s_nt     = 0;
        s_kmin   = 0xffffffffu;
        s_kmax   = 0u;
    }
    const bool general = __syncthreads_or(over) || N > FINAL_CAND_MAX;
    int        k;
    if (general) {
        /* some chunk had more candidates than it may hand on (long runs of equal values,
         * masked rows): select over the whole row instead */
        k = topk_row_general<NV, PEN>(rv, row, a.k, s_pack, TOPK_FAST_MAX, s_cnt16, s_gs);
    } else {
        /* gather every candidate of the row into LDS; one global round trip */
        uint32_t kmin = 0xffffffffu, kmax = 0u;
        for (int i = tid; i < N; i += TPB) {
            int lo = 0, hi = C; /* s_off[lo] <= i < s_off[hi] */
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (s_off[mid] <= i)
                    lo = mid;
                else
                    hi = mid;
            }
            const uint64_t p = a.cand_pack[((long) row * C + lo) * a.cap + (i - s_off[lo])];
            s_cpack[i]       = p;
            const uint32_t key = best_key(p);
            kmin = key < kmin ? key : kmin;
            kmax = key > kmax ? key : kmax;
        }
        kmax = wave_max_u32(kmax);
        kmin = ~wave_max_u32(~kmin);
        if ((tid & (WAVE - 1)) == 0) {
            atomicMax(&s_kmax, kmax);
            atomicMin(&s_kmin, kmin);
        }
        s_gs.hist[tid] = 0;
        __syncthreads();
        k = a.k < N ? a.k : N;
        /* one 8-bit radix step on the highest bits in which the candidates differ */
        const uint32_t diff = s_kmin ^ s_kmax;
        int            sh   = diff ? (31 - __clz((int) diff)) - 7 : 0;
        if (sh < 0)
            sh = 0;
        for (int i = tid; i < N; i += TPB)
            atomicAdd(&s_gs.hist[(best_key(s_cpack[i]) >> sh) & 255u], 1);
        __syncthreads();
        int            remaining = k;
        const int      digit     = radix_pick_digit(s_gs.hist, remaining, s_gs.scan, s_gs.sel);
        const uint32_t low       = ((s_kmax >> sh) & ~255u) | (uint32_t) digit;
        /* everything in or above the digit that holds the k-th largest */
        for (int i = tid; i < N; i += TPB) {
            const uint64_t p = s_cpack[i];
            if ((best_key(p) >> sh) >= low) {
                const int pos = atomicAdd(&s_n, 1);
                if (pos < TPB)
                    s_m[pos] = p;
            }
        }
        __syncthreads();
        const int m = s_n;
        if (m <= TPB) {
            /* order them by counting (entries are distinct); the first k are the survivors */
            uint64_t me   = 0;
            int      rank = 0;
            if (tid < m) {
                me = s_m[tid];
                for (int j = 0; j < m; ++j)
                    rank += s_m[j] > me;
                if (rank < k)
                    s_pack[rank] = me;
            }
            __syncthreads();
        } else {
            /* crowded digit (many near-equal candidates): full radix select in LDS */
            if (tid == 0)
                s_n = 0;
            int            need_ties;
            const uint32_t kth =
                lds_kth_largest(s_cpack, N, k, s_gs.hist, s_gs.scan, s_gs.sel, need_ties);
            for (int i = tid; i < N; i += TPB)
                if (best_key(s_cpack[i]) == kth)
                    atomicAdd(&s_nt, 1);
            __syncthreads();
            const int n_ties = s_nt;
            for (int i = tid; i < N; i += TPB) {
                const uint64_t p    = s_cpack[i];
                const uint32_t key  = best_key(p);
                bool           take = key > kth;
                if (key == kth) {
                    take = true;
                    if (n_ties > need_ties) { /* only the lowest-index ties survive */
                        int rank = 0;
                        for (int j = 0; j < N; ++j)
                            rank += (best_key(s_cpack[j]) == kth) && (s_cpack[j] > p);
                        take = rank < need_ties;
                    }
                }
                if (take) {
                    const int pos = atomicAdd(&s_n, 1);
                    s_m[pos]      = p; /* k <= TOPK_FAST_MAX <= TPB entries */
                }
            }
            __syncthreads();
            uint64_t me   = 0;
            int      rank = 0;
            if (tid < k) {
                me = s_m[tid];
                for (int j = 0; j < k; ++j)
                    rank += s_m[j] > me;
                s_pack[rank] = me;
            }
            __syncthreads();
        }
    }
    /* k <= TOPK_FAST_MAX = 128: the tail runs on one wavefront without barriers */
    if (tid < WAVE) {
        const int tok =
            finish_sorted_wave(k, s_pack, a.inv_t, a.top_p, a.min_p, u_row, s_fs.tab);
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
                                                     float *__restrict__ probs, long ld_probs) {
    __shared__ __align__(16) uint32_t s_cnt16[PEN ? NV * TPB * 2 : 1];
    __shared__ uint64_t s_red[NWAVES];
    __shared__ uint64_t s_tab[32];
    __shared__ double   s_total;
    const int           row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
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
    fetch_chunk<NV, PEN>(rv, row, base, end, s_cnt16, v);
    const float  mx  = key2f(best_key(row_best_from_chunks(chunk_best, row, rv.n_chunks, s_red)));
    const double tot = s_total;
    float       *out = probs + (long) row * ld_probs;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int e = base + 4 * (j * TPB + tid);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            if (e + c < end) {
                const float p = geist_expf_glibc(softmax_arg(f4_get(v[j], c), mx, inv_t), s_tab);
                out[e + c]    = (float) ((double) p / tot);
            }
        }
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
    history_clear<NV * TPB * 4>(s_cnt16);
    history_count(rv, row, base, end, s_cnt16);
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
                    rowp[e] = penalise(rowp[e], cnt[c], rv.rep, rv.freq, rv.pres);
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

void launch_chunk_best(const Launch &L, uint64_t *chunk_best) {
    const dim3 grid(L.rv.n_chunks, L.rows), block(TPB);
    dispatch(L.nv, L.pen, [&](auto nv, auto pen) {
        k_chunk_best<GS_NV, GS_PEN><<<grid, block, 0, L.stream>>>(L.rv, chunk_best);
    });
}

void launch_chunk_expsum(const Launch &L, float inv_t, const uint64_t *chunk_best,
                         double *chunk_sum, const int32_t *probe_token, float *probe_p) {
    const dim3 grid(L.rv.n_chunks, L.rows), block(TPB);
    dispatch(L.nv, L.pen, [&](auto nv, auto pen) {
        k_chunk_expsum<GS_NV, GS_PEN><<<grid, block, 0, L.stream>>>(L.rv, inv_t, chunk_best,
                                                                    chunk_sum, probe_token, probe_p);
    });
}

void launch_topk_scan(const Launch &L, int k, int cap, uint64_t *cand_pack, int32_t *cand_cnt) {
    const dim3 grid(L.rv.n_chunks, L.rows), block(TPB);
    dispatch(L.nv, L.pen, [&](auto nv, auto pen) {
        k_topk_scan<GS_NV, GS_PEN><<<grid, block, 0, L.stream>>>(L.rv, k, cap, cand_pack, cand_cnt);
    });
}

void launch_row_final(const Launch &L, const FinalLaunch &f) {
    FinalArgs a;
    a.mode       = f.mode;
    a.k          = f.k;
    a.cap        = f.cap;
    a.inv_t      = f.inv_t;
    a.top_p      = f.top_p;
    a.min_p      = f.min_p;
    a.uniforms   = f.uniforms;
    a.chunk_best = f.chunk_best;
    a.chunk_sum  = f.chunk_sum;
    a.cand_pack  = f.cand_pack;
    a.cand_cnt   = f.cand_cnt;
    a.out        = f.out;
    const dim3 grid(L.rows), block(TPB);
    dispatch(L.nv, L.pen, [&](auto nv, auto pen) {
        k_row_final<GS_NV, GS_PEN><<<grid, block, 0, L.stream>>>(L.rv, a);
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
                        const double *chunk_sum, float *probs, long ld_probs) {
    const dim3 grid(L.rv.n_chunks, L.rows), block(TPB);
    dispatch(L.nv, L.pen, [&](auto nv, auto pen) {
        k_write_probs<GS_NV, GS_PEN><<<grid, block, 0, L.stream>>>(L.rv, inv_t, chunk_best,
                                                                   chunk_sum, probs, ld_probs);
    });
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
