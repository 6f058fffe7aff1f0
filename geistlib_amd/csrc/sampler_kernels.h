/*
 * sampler_kernels.h -- host-visible launch interface of the sampling kernels.
 */
#ifndef GEIST_SAMPLER_KERNELS_H
#define GEIST_SAMPLER_KERNELS_H

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gs {

constexpr int MAX_CHUNKS     = 128;  /* chunks per row */
constexpr int TMAX_LDS       = 8192; /* thread maxima of one row the final kernel holds in LDS */
constexpr int SEL_MAX        = 192;  /* threads whose elements the final kernel re-reads */
constexpr int TOPK_FAST_MAX  = 128;  /* largest k served by the candidate path */
constexpr int TOPK_MAX       = 8192; /* the reference caps top_k here (sampler.c:213-215) */
constexpr int HISTORY_MAX    = 65535;

enum { FINAL_ARGMAX = 0, FINAL_TEMPERATURE = 1, FINAL_TOPK = 2, FINAL_SORTED = 3 };

/* One batch of logit rows as the kernels see it, with the transform applied while reading. */
struct RowView {
    const float   *logits; /* row 0 */
    long           ld;
    int            n_vocab;
    int            per_chunk;
    int            n_chunks;
    int            vec_ok; /* rows are 16-byte aligned: float4 loads allowed */
    int            stream_loads; /* this pass is the last to read the rows and they come from HBM:
                                    non-temporal loads */
    const int32_t *hist;   /* NULL = no penalties */
    long           hist_ld;
    const int32_t *hist_len;
    float          rep, freq, pres;
    double         inv_rep; /* 1.0 / (double) rep, see penalise() */
    float          softcap; /* 0 = off */
    int            n_rows; /* rows of the batch (hist_len has that many entries) */
    const uint32_t *allowed;   /* NULL = no mask; bit e of a row's mask set = token e allowed */
    long            allowed_ld; /* words between rows, 0 = one mask for all rows */
};

/* Where the workgroups of a row meet in the one-pass exp-sum kernel (k_scan_expsum): one 64-bit
 * slot per (row, chunk), zero until the chunk's workgroup stores its packed maximum there (never
 * zero). Two such arrays take turns from launch to launch: a launch finds its own array all
 * zero and zeroes the slots that the launch before it used in the other. */
constexpr int ARRIVE_STRIDE_INTS = 32; /* a cache line of its own for every row's counter */
struct MeetSpace {
    uint64_t *slots;       /* [rows * n_chunks] of this launch, zero on entry */
    uint64_t *stale;       /* the slots of the launch before, zeroed by this one */
    uint32_t  stale_count;
    uint32_t  wait_limit;  /* polls before a workgroup reads the row for itself; 0 = do not wait */
    uint32_t  local;       /* the workgroups that meet run on one XCD (the grid deals a row's
                            * workgroups to one, and the device was seen to place them so): a slot
                            * is written with a plain store, which that XCD's L2 holds and serves
                            * to the polls -- a device-scope store is written through to memory
                            * first (a meeting of 63 workgroups: 0.6 against 2.5 us). Should the
                            * workgroups not share an XCD after all, the polls never see the slot,
                            * the bounded wait runs out and each workgroup reads the row itself. */
};

/* Where a sampling step reports that the ids of all its rows are written: `epoch` goes into
 * *h_done (page-locked host memory) after them. h_done == NULL: nobody is told. `rows_done` is a
 * zeroed device counter that the one-launch top-k kernel leaves zeroed (its rows finish in any
 * order; the last one reports). */
struct Notify {
    uint64_t *h_done;
    uint64_t  epoch;
    uint32_t *rows_done;
};
/* a small fill kernel: n 64-bit words at p become zero (recorded into HIP graphs in place of a
 * memset node) */
void launch_zero_words(hipStream_t stream, uint64_t *p, uint32_t n);
/* the same report from a launch of its own, for the steps whose last kernel does not make it */
void launch_publish_epoch(hipStream_t stream, const Notify &nt);

struct Launch {
    RowView     rv;
    int         rows;
    int         nv;  /* float4 groups per thread: 2 or 8 */
    bool        pen; /* history lookup on */
    hipStream_t stream;
};

/* Workspace of the candidate path of the full-vocabulary top-p / min-p modes. Elements are
 * binned by z = (max - l) * inv_t in steps of 1/ZBIN_PER_NAT; a row the thread-maxima shortcut
 * cannot serve derives (from the binned mass of its thread maxima and from min_p) the last bin
 * that can hold an element of its kept prefix, a third pass over the row lists the elements up
 * to that bin with their normalised probabilities, and a row-final kernel works on the list. */
constexpr int ZBINS        = 128;
constexpr int ZBIN_PER_NAT = 4;
constexpr int CAND_CAP     = 16384; /* list entries per row */
constexpr int CAND_LDS     = 4096;  /* lists up to this length are staged in LDS */
constexpr int CAND_COUNT_STRIDE = 32;
struct CandSpace {
    int32_t  *row_bound; /* [rows] last z bin listed */
    uint32_t *out_key;   /* [rows] bits of a pn no element past that bin can exceed */
    uint32_t *key;       /* [rows][CAND_CAP] bits of pn */
    uint32_t *idx;       /* [rows][CAND_CAP] vocabulary ids */
    int32_t  *count;     /* [rows * CAND_COUNT_STRIDE]: a row's counter has a cache line to itself
                          * (the appending wavefronts' atomic adds to one line serialise) */
    double   *row_sum;   /* [rows] the row's exp-sum, for lists that hold p instead of pn */
    int32_t  *path;      /* [rows] which walk served the row: 1 thread-maxima shortcut, 2 list,
                          * 3 whole row */
};

/* Workspace of the candidate path of the top-k modes: what each scanning wavefront hands on to
 * the row-final kernel. A row is scanned by n_chunks * 4 wavefronts; wavefront w of row r owns
 * CAND_GROUPS slots. */
constexpr int NWAVES_PER_CHUNK = 4; /* a chunk is scanned by one workgroup of four wavefronts */
constexpr int CAND_SLOTS     = 32;  /* float4 groups a wavefront has room for ... */
constexpr int CAND_GROUPS    = 32;  /* ... and how many it may hand on */
constexpr int CAND_CHUNKS_MAX = 32; /* rows of up to 32 chunks of 8192 logits take this path */
constexpr int CAND_K_MAX     = 64;  /* largest k: the survivors are ordered one per lane */
constexpr int CAND_LANES_MAX = 16;  /* largest `m` (see k_cand_scan) that leaves room in the slots */
struct WaveCands {
    float4   *val;   /* [rows][waves][CAND_SLOTS] the groups */
    int32_t  *idx;   /* [rows][waves][CAND_SLOTS] index of each group's first element, -1 = unused */
    uint32_t *bound; /* [rows][waves] key of the wavefront's bound T; 0xffffffff = it had too many
                      * groups and handed none on */
};
/* bytes of the three arrays for `row_waves` = rows * waves per row */
inline size_t wave_cands_bytes(size_t row_waves) {
    return row_waves * (CAND_SLOTS * (sizeof(float4) + sizeof(int32_t)) + 8); /* 648 */
}
inline WaveCands wave_cands_at(void *base, size_t row_waves) {
    WaveCands w;
    w.val   = static_cast<float4 *>(base);
    w.idx   = reinterpret_cast<int32_t *>(w.val + row_waves * CAND_SLOTS);
    w.bound = reinterpret_cast<uint32_t *>(w.idx + row_waves * CAND_SLOTS);
    return w;
}
/* What the wavefronts of the one-launch form of that path (k_cand_scan_final) hand on to the
 * workgroup that finishes the row: per scanning wavefront (16 per workgroup, G workgroups per row)
 * OL_SLOTS float4 groups -- those that hold an element at or above the workgroup's bound T_w --
 * with the index of each group's first element, and their number (more than OL_SLOTS: it had too
 * many and the row cannot be certified) beside the key of T_w. */
constexpr int OL_TOP      = 8;   /* maxima a wavefront enters for its workgroup's bound */
constexpr int OL_SLOTS    = 16;  /* groups a scanning wavefront may hand on */
constexpr int OL_WG_MAX   = 8;   /* workgroups per row (CAND_CHUNKS_MAX chunks, four each) */
constexpr int OL_RANK_MAX = 64;  /* largest rank `r` of the workgroup's bound the path is used for */
struct WgCands {
    float4   *val;   /* [rows][OL_SLOTS][G * 16] the float4 groups */
    uint32_t *idx;   /* [rows][OL_SLOTS][G * 16] index of each group's first element */
    uint32_t *count; /* [rows][G][16] key of T_w (its sixteen leading bits) | number of groups */
};
inline size_t wg_cands_bytes(size_t rows, size_t wgs_per_row) {
    return rows * wgs_per_row * (16 * OL_SLOTS * 20 + 16 * sizeof(uint32_t));
}
inline WgCands wg_cands_at(void *base, size_t rows, size_t wgs_per_row) {
    WgCands w;
    w.val   = static_cast<float4 *>(base);
    w.idx   = reinterpret_cast<uint32_t *>(w.val + rows * wgs_per_row * 16 * OL_SLOTS);
    w.count = w.idx + rows * wgs_per_row * 16 * OL_SLOTS;
    return w;
}
/* `r` for a workgroup that holds `elems` of a row's n_vocab logits, of which about k_eff lead:
 * the smallest rank such that the workgroup holding that many of the k_eff is a one-in-10^8 event
 * when the logits' order is unrelated to the vocabulary's (all of them when it holds the whole
 * row). 0 = the one-launch form does not pay (r would exceed OL_RANK_MAX). */
int cand_rank_for(int k_eff, size_t n_vocab, size_t elems);

/* The final stage of that path keeps its candidates (at most 16 x 64 ids) in an open-addressing
 * table of HT_SLOTS slots in LDS and looks the row's token history up in it. */
constexpr int HT_SLOTS       = 4096;

/* `m` for a row of n_vocab logits of which about k_eff lead: the smallest number of lanes such
 * that a wavefront (2048 logits) holding that many of the k_eff is a one-in-10^8 event when the
 * logits' order is unrelated to the vocabulary's. 0 = the candidate path does not pay
 * (m would exceed CAND_LANES_MAX). */
int cand_lanes_for(int k_eff, size_t n_vocab);

struct FinalLaunch {
    CandSpace       cand;
    bool            minp_listed; /* the exp-sum pass already listed the rows under the min-p bound */
    bool            minp_direct; /* ... and the list walk runs straight after it: no row-final
                                    kernel, no listing pass; a row whose list overflowed goes to
                                    the whole-row walk */
    int             mode, k, k_sel;
    bool            cap_after; /* top-k: the scan ran before the soft-cap, the row-final kernel
                                  applies it to what it keeps */
    float           inv_t, top_p, min_p;
    const float    *uniforms;
    const uint64_t *chunk_best;
    const double   *chunk_sum;
    const double   *slab_sum;
    const float    *tmax;
    int32_t        *out;
    int32_t        *row_flag;
};

/* The one pass over the rows of the modes that weigh every element (k_scan_expsum): tmax and
 * chunk_best as launch_tmax_scan writes them, and chunk_sum[row][chunk], the sum of
 * expf((l - max) * inv_t) over the chunk in double.
 * probe_token != NULL: the rows are n_seq * (probe_L + 1) target rows of a speculative batch and
 * probe_token holds the n_seq * probe_L draft ids; probe_p[row] receives p at the row's draft id.
 * list != NULL (min-p set): the pass also lists, per row, every element up to z bin zb_list with
 * its softmax argument -- the min-p bound needs nothing but the row maximum (the pass clears
 * list->count itself).
 * slab_sum != NULL (and no list): also the sums of the chunk's slabs of 1024 elements,
 * [rows][chunks][8], which the index-order walks locate their starting point with.
 * fast: the weights of the sums from the hardware's 2^z (relative error about 1e-7) instead of
 * the bit-exact expf; p at the probed token stays exact. Without penalties and without a list
 * the workgroups of a row then do not meet: each sums against its chunk's maximum and a second,
 * small launch scales the sums to the row's (k_rescale_sums).
 * Returns 0 or a hipError_t value (the launch itself is checked by the caller as usual). */
int launch_scan_expsum(const Launch &L, float inv_t, float *tmax, uint64_t *chunk_best,
                       double *chunk_sum, const int32_t *probe_token, int probe_L, float *probe_p,
                       const CandSpace *list, int zb_list, double *slab_sum, const MeetSpace &meet,
                       bool fast = false);
/* The temperature draw in one kernel (sampler_draw.h): out[row] = the id drawn with
 * uniforms[row]. For L.nv == 2. `meet.slots` holds 2 * rows * n_chunks zeroed words: the
 * workgroups of a row meet twice. */
void launch_temperature_draw(const Launch &L, float inv_t, const float *uniforms, int32_t *out,
                             const MeetSpace &meet);
/* last z bin that can hold an entry passing min_p (with slack); ZBINS - 1 when min_p is off or
 * that deep */
int zbin_of_min_p(float min_p);

struct SpecLaunch {
    int             n_seq, L, greedy;
    float           inv_t;
    const float    *q;
    long            ld_q;
    const int32_t  *draft;
    const float    *uniforms;
    const uint64_t *chunk_best;
    const double   *chunk_sum;
    const float    *probe_p;
    double         *resid_sum;
    double         *resid_slab; /* [n_seq][chunks][8] */
    const double   *slab_sum;   /* [rows][chunks][8] from the exp-sum pass */
    void           *verdict; /* [n_seq] x SPEC_VERDICT_BYTES, written by the acceptance kernel */
    int32_t        *out_tokens;
    int32_t        *n_accepted;
};
constexpr int SLABS_MAX         = 8; /* slab sums are stored 8 per chunk whatever NV is */
constexpr int SPEC_DRAFT_MAX      = 63;
constexpr int NGRAM_SUFFIX_MAX    = 8;  /* session.c:455-456 */
constexpr int NGRAM_DRAFT_MAX     = 16; /* GEIST_SPEC_KMAX_HARDCAP, session.c:515 */
constexpr int SPEC_VERDICT_BYTES = 24;
/* meet != NULL (stochastic verification only): the residual sums and the draw in one launch (the
 * workgroups of a sequence wait for one another); NULL: two launches */
void launch_spec(const Launch &L, const SpecLaunch &sp, const MeetSpace *meet = nullptr);
constexpr int SPEC_ONE_LAUNCH_WGS_PER_CU = 2; /* what the one-launch kernel's 171 registers allow */
/* chunk_best may be NULL when only the thread maxima are wanted */
void launch_tmax_scan(const Launch &L, float *tmax, uint64_t *chunk_best,
                      int32_t *zero_per_row = nullptr);
void launch_row_final(const Launch &L, const FinalLaunch &f);
/* the candidate path of top-k (sampler_cands.h): L.nv == 8, no soft-cap, no mask, 16-byte aligned
 * rows of at most CAND_CHUNKS_MAX chunks; the scan reads the logits raw (penalties are the final
 * kernel's) and also stores the thread maxima */
void launch_cand_scan(const Launch &L, float *tmax, const WaveCands &wc, int m);
void launch_final_cand(const Launch &L, const FinalLaunch &f, const WaveCands &wc);
/* both in one launch (k_cand_scan_final): `arrive` holds one zeroed counter per row,
 * ARRIVE_STRIDE_INTS apart, and is left zeroed; `tmax` receives the thread maxima of the rows that
 * fall back to the slower paths. r_w / r_last: the rank of the bound of a full workgroup and of
 * the row's last one (cand_rank_for). far_always: read the hand-over with agent-scope loads whatever
 * the placement of the row's workgroups (for tests of that branch). */

/* *same_xcd: workgroups of a grid whose linear ids are equal modulo 8 run on one XCD (and so
 * share an L2): then launch_cand_scan_final hands a row over through that L2. Runs a small
 * kernel and waits for it. Returns a hipError_t value. */
int probe_workgroup_placement(hipStream_t stream, bool *same_xcd);
void launch_cand_scan_final(const Launch &scan, const Launch &L, const FinalLaunch &f, float *tmax,
                            const WgCands &wc, int r_w, int r_last, uint32_t *arrive,
                            bool far_always, const Notify &nt, int wgs_per_row, int groups);
/* returns a hipError_t value */
int  launch_topk_general(const Launch &L, const FinalLaunch &f);
/* Per-device kernel attributes; call once with the device current. Returns a hipError_t value. */
int configure_device_kernels();
/* rows flagged 1 by the sorted row-final kernel: list their candidates, then draw from the
 * list; rows the list cannot serve (and rows the row-final kernel flagged 2) take the whole-row
 * walk in the same launch: probabilities of the whole row into `probs`, then the walk over them */
/* The whole-row walk spread over the workgroups of the row's chunks (sampler_walk_coop.h), for
 * the rows the list walk flags 2 when `spread` is set: `rows` is the workspace of
 * walk_coop_bytes(max rows) bytes, zero before its first use and cleared again by this call when
 * `clear` is set; the steps of this launch are numbered from step_base + 1 on (at most 16); `hint`
 * (two words of page-locked host memory, or null): a launch in which a row was walked in full
 * writes the call's number `call` to word 0, one in which a wait ran out (the workspace then has
 * to be cleared) to word 1. */
struct WalkCoop {
    void     *rows;
    bool      spread;
    bool      clear;
    uint32_t  step_base;
    uint32_t  wait_limit;
    uint32_t *hint;
    uint32_t  call;
};
size_t walk_coop_bytes(size_t rows);
void launch_candidates(const Launch &L, const FinalLaunch &f, float *probs, long ld_probs,
                       const WalkCoop &wc);
/* row_flag != NULL: only rows flagged 2 are written */
void launch_write_probs(const Launch &L, float inv_t, const uint64_t *chunk_best,
                        const double *chunk_sum, float *probs, long ld_probs,
                        const int32_t *row_flag);
/* after launch_tmax_scan(L, tmax, chunk_best): out[row][j] = log_softmax(row)[tokens[row][j]] */
void launch_logprob(const Launch &L, const uint64_t *chunk_best, double *chunk_sum,
                    const int32_t *tokens, long tokens_ld, int k_per_row, double *out, long out_ld);
void launch_ngram_draft(hipStream_t stream, const int32_t *history, long history_ld,
                        const int32_t *history_len, const int32_t *seeds, int n_seq, int k_max,
                        int max_suffix, int32_t *out, long out_ld, int32_t *out_count,
                        int32_t *out_match);
void launch_penalties(const Launch &L, float *logits_rw);
void launch_rng_units(hipStream_t stream, uint64_t *states, int shared, int rows, float *uniforms);

} // namespace gs
#endif
