/*
 * sampler_abi.hip -- the C ABI declared in include/geist_sampler_hip.h: argument checks, launch
 * geometry and the order of kernels for each sampling configuration. No arithmetic on logits
 * happens on the host.
 */
#include "../../include/geist_sampler_hip.h"

#include <hip/hip_runtime.h>

#include <pthread.h>
#include <time.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <new>
#include <algorithm>
#include <vector>

#include "../../include/geist_lm_head_hip.h"
#include "lm_head_kernels.h"
#include "spec_head_kernels.h"
#include "sampler_kernels.h"
#include "sampler_host.h"

using namespace gs;

/* Host side of gs::MeetSpace: the two slot arrays ([max_rows * max_chunks] each, zeroed when
 * made), how many slots the last launch on each array used, and whose turn it is. */
struct MeetState {
    uint64_t *slots[2] = {nullptr, nullptr};
    uint64_t *recorded = nullptr; /* a third array, for launches recorded into a HIP graph: a graph
                                   * is replayed with the arguments it was recorded with, so the
                                   * turns of the two arrays above mean nothing to it */
    uint32_t  used[2]  = {0, 0};
    int       turn     = 0;
    uint32_t  capacity = 0;     /* slots per array */
    bool      suspect  = false; /* a launch failed after the bookkeeping: zero both arrays */
};

struct geist_hip_sampler {
    int         device     = 0;
    hipStream_t stream     = nullptr;
    size_t      max_rows   = 0;
    size_t      max_vocab  = 0;
    int         max_chunks = 0;

    /* device workspace */
    uint64_t *chunk_best = nullptr; /* [max_rows][max_chunks] */
    int32_t   *row_arrive = nullptr; /* per row: how many of its workgroups have scanned (k_cand_scan_final) */
    int        fused_wg_limit = 0;   /* largest grid that kernel is used for */
    /* geist_hip_sampler_notify_ids: every sampling call reports when its ids are written */
    bool       notify = false;
    uint64_t  *h_done = nullptr;     /* page-locked: the epoch of the last call whose ids are written */
    uint64_t   epoch = 0;            /* of the last call enqueued */
    uint32_t  *rows_done = nullptr;  /* device counter of the one-launch top-k kernel */
    bool       epoch_by_kernel = false; /* the call being enqueued reports from its own kernel */
    bool       tell = false;            /* the call being enqueued reports at all */
    uint32_t   wait_spin_us = 2000;  /* geist_hip_sampler_wait_ids: how long it watches the word */
    bool       fast_sums = false;    /* geist_hip_sampler_set_sums */
    bool       handoff_far = false;  /* that kernel reads the hand-over with agent-scope loads
                                      * whatever the placement (geist_hip_sampler_handoff_scope) */
    bool       spec_one_launch = true; /* residual sums and draw of spec verification in one launch */
    int        cu_count = 0;
    int        fused_wg_default = 0; /* ... as the device allows */
    MeetState  meet_own;             /* where the workgroups of the one-pass exp-sum kernel meet */
    MeetState *meet      = &meet_own; /* (the allocation-free entry point shares one per device) */
    uint32_t  wait_limit = 1u << 16; /* polls a workgroup of that kernel waits for its row */
    double   *chunk_sum  = nullptr; /* [max_rows][max_chunks] */
    double   *resid_sum  = nullptr; /* [max_rows][max_chunks] spec verification */
    double   *slab_sum   = nullptr; /* [max_rows][max_chunks][8] slab sums of the exp-sum pass */
    double   *resid_slab = nullptr; /* [max_rows][max_chunks][8] spec verification */
    void     *verdict    = nullptr; /* [max_rows] acceptance results of spec verification */
    float    *tmax       = nullptr; /* [max_rows][max_chunks][256] per-thread maxima */
    void     *wcands     = nullptr; /* what the top-k scan's wavefronts hand on (WaveCands) */
    size_t    wcands_row_waves = 0; /* (row, wavefront) pairs it has room for */
    int32_t  *row_flag   = nullptr; /* [max_rows] */
    float    *uniforms   = nullptr; /* [max_rows] */
    float    *probe_p    = nullptr; /* [max_rows] */
    int32_t  *scalar_out = nullptr; /* [max_rows] */
    int32_t  *h_scalar   = nullptr; /* pinned */
    float    *probs      = nullptr; /* [max_rows][max_vocab], allocated on first use by the
                                     * full-vocabulary top-p / min-p path */
    gs::CandSpace cand   = {};      /* candidate lists of that path, allocated with probs */
    void     *walk_rows  = nullptr; /* workspace of the whole-row walk spread over the row's
                                     * chunks (sampler_walk_coop.h), allocated with probs */
    uint32_t *walk_hint  = nullptr; /* pinned, two words: the number of the last call in which
                                     * a row was walked in full / in which a wait ran out */
    uint32_t  walk_steps = 0;       /* step numbers handed out so far */
    uint32_t  walk_calls = 0;       /* calls of the top-p / min-p path so far */
    uint32_t  walk_cleared = 0;     /* ... the one before which the workspace was last cleared */
    int       walk_mode  = 0;       /* geist_hip_sampler_set_whole_row_walk */
    bool      walk_clear = false;   /* clear the workspace before its next use */
    void    *q6k_ws      = nullptr; /* scratch of the Q6_K projection, sized like f64_ws */
    size_t   q6k_in = 0, q6k_out = 0;
    void    *f64_ws      = nullptr; /* scratch of the f64 projection for n_in <= f64_in and
                                     * n_out <= f64_out, allocated on first use */
    size_t   f64_in = 0, f64_out = 0;

    size_t topk_paths_rows  = 0;     /* rows of the last top-k call that took the candidate path */ /* see geist_hip_sampler_time_stream_kernel */
    bool logits_streamed    = false; /* see geist_hip_sampler_set_logits_hint */
    bool projection_portable = false; /* see geist_hip_sampler_set_projection */
    bool projection_avx2     = false; /* the x86 backend on a host without AVX-512 */
    bool tmax_ready         = false; /* the projection has written the top-k scan's thread maxima
                                        for the rows about to be sampled */

    char err[512] = {0};
};

static int fail(geist_hip_sampler *s, int code, const char *fmt, ...) {
    if (s) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(s->err, sizeof s->err, fmt, ap);
        va_end(ap);
    }
    return code;
}

#define HIPCHK(s, call)                                                                        \
    do {                                                                                       \
        hipError_t e_ = (call);                                                                \
        if (e_ != hipSuccess)                                                                  \
            return fail((s), e_ == hipErrorOutOfMemory ? GEIST_HIP_E_OOM : GEIST_HIP_E_BACKEND, \
                        "%s: %s", #call, hipGetErrorString(e_));                               \
    } while (0)

static int after_launch(geist_hip_sampler *s, const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        if (s->meet)
            s->meet->suspect = true; /* the slots may not be what the bookkeeping says */
        return fail(s, GEIST_HIP_E_BACKEND, "launch of %s failed: %s", what, hipGetErrorString(e));
    }
    return GEIST_HIP_OK;
}

/* ---- launch geometry ---------------------------------------------------------------------- */
static bool plan_chunks(size_t rows, size_t n_vocab, int &nv, int &per_chunk, int &n_chunks) {
    const size_t big   = (n_vocab + 8191) / 8192;
    const size_t small = (n_vocab + 2047) / 2048;
    if (big > (size_t) MAX_CHUNKS)
        return false;
    /* fewer than two workgroups per compute unit: cut the rows finer */
    nv                 = (rows * big < 512 && small <= (size_t) MAX_CHUNKS) ? 2 : 8;
    /* every chunk but the last is exactly what one workgroup holds in registers */
    per_chunk = 1024 * nv;
    n_chunks  = (int) ((n_vocab + per_chunk - 1) / per_chunk);
    return true;
}

static int make_launch(geist_hip_sampler *s, const struct geist_hip_rows *r,
                       const struct geist_hip_sample_params *p, bool stochastic, Launch &L) {
    if (!s || !r || !r->d_logits)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null sampler, rows or logits");
    if (r->rows == 0 || r->n_vocab == 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "empty batch (rows=%zu, n_vocab=%zu)", r->rows,
                    r->n_vocab);
    if (r->rows > s->max_rows || r->n_vocab > s->max_vocab)
        return fail(s, GEIST_HIP_E_INVALID_ARG,
                    "batch %zu x %zu exceeds the workspace (%zu x %zu)", r->rows, r->n_vocab,
                    s->max_rows, s->max_vocab);
    if (r->ld < r->n_vocab)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "row stride %zu < n_vocab %zu", r->ld, r->n_vocab);
    if (r->n_vocab > 0x7fffff00u)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "n_vocab too large");
    int nv, per, nc;
    if (!plan_chunks(r->rows, r->n_vocab, nv, per, nc) || nc > s->max_chunks)
        return fail(s, GEIST_HIP_E_UNSUPPORTED, "n_vocab %zu needs more than %d chunks",
                    r->n_vocab, s->max_chunks);
    const bool pen = p && r->d_history && r->d_history_len &&
                     (p->repetition_penalty != 1.0f || p->frequency_penalty != 0.0f ||
                      p->presence_penalty != 0.0f);
    if (pen && r->history_ld > (size_t) HISTORY_MAX)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "history_ld %zu exceeds %d", r->history_ld,
                    HISTORY_MAX);
    if (pen && !(p->repetition_penalty > 0.0f))
        return fail(s, GEIST_HIP_E_INVALID_ARG, "repetition_penalty must be > 0");
    if (r->d_allowed && r->allowed_ld != 0 && r->allowed_ld < (r->n_vocab + 31) / 32)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "allowed_ld %zu < %zu mask words per row",
                    r->allowed_ld, (r->n_vocab + 31) / 32);
    L.rv.logits    = r->d_logits;
    L.rv.ld        = (long) r->ld;
    L.rv.n_vocab   = (int) r->n_vocab;
    L.rv.per_chunk = per;
    L.rv.n_chunks  = nc;
    L.rv.vec_ok    = (((uintptr_t) r->d_logits) % 16 == 0) && (r->ld % 4 == 0);
    L.rv.stream_loads = 0; /* set by the flows for their last pass over the rows */
    L.rv.hist      = pen ? r->d_history : nullptr;
    L.rv.hist_ld   = (long) r->history_ld;
    L.rv.hist_len  = pen ? r->d_history_len : nullptr;
    L.rv.rep       = pen ? p->repetition_penalty : 1.0f;
    L.rv.inv_rep   = 1.0 / (double) L.rv.rep;
    L.rv.freq      = pen ? p->frequency_penalty : 0.0f;
    L.rv.pres      = pen ? p->presence_penalty : 0.0f;
    /* the soft-cap is monotone, so greedy rows skip it (head.c:145-149) */
    L.rv.softcap   = (p && stochastic && p->logit_softcap > 0.0f) ? p->logit_softcap : 0.0f;
    L.rv.n_rows     = (int) r->rows;
    L.rv.allowed    = r->d_allowed;
    L.rv.allowed_ld = (long) r->allowed_ld;
    L.rows         = (int) r->rows;
    L.nv           = nv;
    L.pen          = pen;
    L.stream       = s->stream;
    return GEIST_HIP_OK;
}


/* ---- sampling without any allocation --------------------------------------------------------
 * The workspace of geist_hip_sample_rows_static: a device array that belongs to the code object,
 * so neither a sampler object nor hipMalloc is needed. In host code `scratch` is only the
 * symbol's host-side stand-in; the device address is looked up once per device with
 * hipGetSymbolAddress and kept in g_static_ws[]. Every GPU holds its own copy of the array. */
namespace {
constexpr size_t STATIC_UNITS = GEIST_HIP_STATIC_MAX_UNITS; /* (row, chunk) pairs */
constexpr size_t STATIC_TMAX  = 0;                                     /* float [units][256]  */
constexpr size_t STATIC_BEST  = STATIC_TMAX + STATIC_UNITS * 256 * 4;  /* u64   [units]       */
constexpr size_t STATIC_CSUM  = STATIC_BEST + STATIC_UNITS * 8;        /* double[units]       */
constexpr size_t STATIC_SLAB  = STATIC_CSUM + STATIC_UNITS * 8;        /* double[units][8]    */
constexpr size_t STATIC_ROW_WAVES = STATIC_UNITS + 512;            /* (row, wavefront) pairs */
constexpr size_t STATIC_WCANDS = STATIC_SLAB + STATIC_UNITS * 8 * 8;   /* WaveCands           */
constexpr size_t STATIC_MEET   = STATIC_WCANDS + STATIC_ROW_WAVES * 648; /* u64 [2][2 units]:
                                                                            the meeting slots,
                                                                            zero when loaded */
constexpr size_t STATIC_BYTES  = STATIC_MEET + 3 * 2 * STATIC_UNITS * 8; /* (the third array: for
                                                                           launches recorded into a
                                                                           HIP graph) */
static_assert(STATIC_MEET % 16 == 0, "64-bit atomics");
static_assert(STATIC_WCANDS % 16 == 0, "float4 slots");
constexpr int    STATIC_MAX_DEVICES = 64;
} // namespace
static __device__ __align__(256) unsigned char scratch[STATIC_BYTES];

static MeetState      g_static_meet[STATIC_MAX_DEVICES]; /* turn and use of its meeting slots */
static unsigned char *g_static_ws[STATIC_MAX_DEVICES]; /* device address of `scratch`, per device */
static bool           g_static_ws_tried[STATIC_MAX_DEVICES];
static hipError_t     g_static_ws_err[STATIC_MAX_DEVICES];
static pthread_mutex_t g_static_ws_lock = PTHREAD_MUTEX_INITIALIZER;

/* The device address of `scratch` on `device` (which must be current). Looked up on the first
 * call per device; later calls return the kept pointer without touching the runtime. */
static hipError_t static_workspace(int device, unsigned char **out) {
    if (device < 0 || device >= STATIC_MAX_DEVICES)
        return hipErrorInvalidDevice;
    pthread_mutex_lock(&g_static_ws_lock);
    if (!g_static_ws_tried[device]) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        g_static_ws_err[device]   = e;
        g_static_ws[device]       = e == hipSuccess ? static_cast<unsigned char *>(p) : nullptr;
        g_static_ws_tried[device] = e == hipSuccess; /* a failed lookup is tried again */
    }
    const hipError_t e = g_static_ws_err[device];
    *out               = g_static_ws[device];
    pthread_mutex_unlock(&g_static_ws_lock);
    return e;
}

/* Whether the device (current) places workgroups as k_cand_scan_final needs; probed on the first
 * call per device. */
static bool g_placement_known[STATIC_MAX_DEVICES], g_placement_same[STATIC_MAX_DEVICES];
static hipError_t placement_of(int device, hipStream_t stream, bool *same) {
    *same = false;
    if (device < 0 || device >= STATIC_MAX_DEVICES)
        return hipSuccess;
    pthread_mutex_lock(&g_static_ws_lock);
    hipError_t e = hipSuccess;
    if (!g_placement_known[device]) {
        bool ok = false;
        e       = (hipError_t) gs::probe_workgroup_placement(stream, &ok);
        if (e == hipSuccess) {
            g_placement_known[device] = true;
            g_placement_same[device]  = ok;
        }
    }
    *same = g_placement_known[device] && g_placement_same[device];
    pthread_mutex_unlock(&g_static_ws_lock);
    return e;
}

/* ============================================================================================ */
/* failure text into a caller's buffer (an entry point without a sampler object has no error slot) */
static int report(char *err, size_t err_len, int code, const char *fmt, ...) {
    if (err && err_len) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(err, err_len, fmt, ap);
        va_end(ap);
    }
    return code;
}

extern "C" {

int geist_hip_sampler_create(int device, size_t max_rows, size_t max_vocab, void *stream,
                             geist_hip_sampler **out) {
    if (!out || max_rows == 0 || max_vocab == 0)
        return GEIST_HIP_E_INVALID_ARG; /* sampler.c:138-140 */
    *out = nullptr;
    int n_dev = 0;
    if (hipGetDeviceCount(&n_dev) != hipSuccess || device < 0 || device >= n_dev)
        return GEIST_HIP_E_BACKEND;
    geist_hip_sampler *s = new (std::nothrow) geist_hip_sampler();
    if (!s)
        return GEIST_HIP_E_OOM;
    s->device    = device;
    s->stream    = (hipStream_t) stream;
    s->max_rows  = max_rows;
    s->max_vocab = max_vocab;
    size_t mc    = (max_vocab + 2047) / 2048;
    if (mc > (size_t) MAX_CHUNKS)
        mc = MAX_CHUNKS;
    if ((max_vocab + 8191) / 8192 > (size_t) MAX_CHUNKS) {
        delete s;
        return GEIST_HIP_E_UNSUPPORTED;
    }
    s->max_chunks = (int) mc;
    const size_t rc = max_rows * mc;
    hipError_t   e  = hipSetDevice(device);
    if (e == hipSuccess) e = (hipError_t) configure_device_kernels();
    if (e == hipSuccess) { /* the address of the static workspace, so that the allocation-free
                            * entry point finds it ready (a failure is reported by that call) */
        unsigned char *ws = nullptr;
        (void) static_workspace(device, &ws);
    }
    if (e == hipSuccess) e = hipMalloc((void **) &s->chunk_best, rc * sizeof(uint64_t));
    if (e == hipSuccess) e = hipMalloc((void **) &s->chunk_sum, rc * sizeof(double));
    for (int t = 0; t < 2; ++t) {
        /* two words per (row, chunk): the one-kernel temperature draw meets twice */
        if (e == hipSuccess) e = hipMalloc((void **) &s->meet_own.slots[t], 2 * rc * sizeof(uint64_t));
        if (e == hipSuccess) e = hipMemsetAsync(s->meet_own.slots[t], 0, 2 * rc * sizeof(uint64_t), s->stream);
    }
    if (e == hipSuccess) e = hipMalloc((void **) &s->meet_own.recorded, 2 * rc * sizeof(uint64_t));
    s->meet_own.capacity = (uint32_t) (2 * rc);
    if (e == hipSuccess)
        e = hipMalloc((void **) &s->row_arrive, max_rows * ARRIVE_STRIDE_INTS * sizeof(int32_t));
    if (e == hipSuccess)
        e = hipMemsetAsync(s->row_arrive, 0, max_rows * ARRIVE_STRIDE_INTS * sizeof(int32_t), s->stream);
    {
        /* the one-launch form of the top-k candidate path hands a row over through the L2 its
         * workgroups share: used only where the device places them as that needs (looked at
         * once per device) */
        int cus = 0;
        if (e == hipSuccess)
            e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device);
        bool same = false;
        if (e == hipSuccess)
            e = placement_of(device, s->stream, &same);
        s->cu_count         = cus;
        s->fused_wg_default = same ? cus : 0; /* one workgroup of 1024 threads per compute unit */
        s->fused_wg_limit   = s->fused_wg_default;
    }
    if (e == hipSuccess) e = hipStreamSynchronize(s->stream);
    if (e == hipSuccess) e = hipMalloc((void **) &s->resid_sum, rc * sizeof(double));
    if (e == hipSuccess) e = hipMalloc((void **) &s->slab_sum, rc * 8 * sizeof(double));
    if (e == hipSuccess) e = hipMalloc((void **) &s->resid_slab, rc * 8 * sizeof(double));
    if (e == hipSuccess) e = hipMalloc((void **) &s->tmax, rc * 256 * sizeof(float));
    {
        const size_t chunks8k = (max_vocab + 8191) / 8192;
        s->wcands_row_waves   = max_rows * NWAVES_PER_CHUNK *
                              (chunks8k < (size_t) CAND_CHUNKS_MAX ? chunks8k : (size_t) CAND_CHUNKS_MAX);
        if (e == hipSuccess) e = hipMalloc(&s->wcands, wave_cands_bytes(s->wcands_row_waves));
    }
    if (e == hipSuccess) e = hipMalloc(&s->verdict, max_rows * SPEC_VERDICT_BYTES);
    if (e == hipSuccess) e = hipMalloc((void **) &s->row_flag, max_rows * sizeof(int32_t));
    if (e == hipSuccess) e = hipMalloc((void **) &s->uniforms, max_rows * sizeof(float));
    if (e == hipSuccess) e = hipMalloc((void **) &s->probe_p, max_rows * sizeof(float));
    if (e == hipSuccess) e = hipMalloc((void **) &s->scalar_out, max_rows * sizeof(int32_t));
    if (e == hipSuccess) e = hipHostMalloc((void **) &s->h_scalar, 64 * sizeof(int32_t), hipHostMallocDefault);
    if (e != hipSuccess) {
        const int code = e == hipErrorOutOfMemory ? GEIST_HIP_E_OOM : GEIST_HIP_E_BACKEND;
        geist_hip_sampler_destroy(s);
        return code; /* sampler.c:142-145 */
    }
    *out = s;
    return GEIST_HIP_OK;
}

void geist_hip_sampler_destroy(geist_hip_sampler *s) {
    if (!s)
        return;
    (void) hipSetDevice(s->device);
    (void) hipStreamSynchronize(s->stream);
    (void) hipFree(s->chunk_best);
    (void) hipFree(s->chunk_sum);
    (void) hipFree(s->row_arrive);
    (void) hipFree(s->rows_done);
    if (s->h_done)
        (void) hipHostFree(s->h_done);
    (void) hipFree(s->meet_own.slots[0]);
    (void) hipFree(s->meet_own.slots[1]);
    (void) hipFree(s->meet_own.recorded);
    (void) hipFree(s->resid_sum);
    (void) hipFree(s->slab_sum);
    (void) hipFree(s->resid_slab);
    (void) hipFree(s->tmax);
    (void) hipFree(s->wcands);
    (void) hipFree(s->verdict);
    (void) hipFree(s->row_flag);
    (void) hipFree(s->uniforms);
    (void) hipFree(s->probe_p);
    (void) hipFree(s->scalar_out);
    (void) hipFree(s->probs);
    (void) hipFree(s->walk_rows);
    if (s->walk_hint)
        (void) hipHostFree(s->walk_hint);
    (void) hipFree(s->f64_ws);
    (void) hipFree(s->q6k_ws);
    (void) hipFree(s->cand.row_bound);
    (void) hipFree(s->cand.out_key);
    (void) hipFree(s->cand.key);
    (void) hipFree(s->cand.idx);
    (void) hipFree(s->cand.count);
    (void) hipFree(s->cand.row_sum);
    (void) hipFree(s->cand.path);
    if (s->h_scalar)
        (void) hipHostFree(s->h_scalar);
    delete s;
}

const char *geist_hip_sampler_last_error(const geist_hip_sampler *s) { return s ? s->err : ""; }

int geist_hip_sampler_sync(geist_hip_sampler *s) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    HIPCHK(s, hipStreamSynchronize(s->stream));
    return GEIST_HIP_OK;
}

int geist_hip_sampler_set_logits_hint(geist_hip_sampler *s, int hint) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (hint != GEIST_HIP_LOGITS_CACHED && hint != GEIST_HIP_LOGITS_STREAMED)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "unknown logits hint %d", hint);
    s->logits_streamed = hint == GEIST_HIP_LOGITS_STREAMED;
    return GEIST_HIP_OK;
}

int geist_hip_sampler_set_projection(geist_hip_sampler *s, int mode) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (mode != GEIST_HIP_PROJECTION_X86 && mode != GEIST_HIP_PROJECTION_PORTABLE &&
        mode != GEIST_HIP_PROJECTION_X86_AVX2)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "unknown projection mode %d", mode);
    s->projection_portable = mode == GEIST_HIP_PROJECTION_PORTABLE;
    s->projection_avx2     = mode == GEIST_HIP_PROJECTION_X86_AVX2;
    return GEIST_HIP_OK;
}

int geist_hip_sampler_set_stream(geist_hip_sampler *s, void *stream) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    s->stream = (hipStream_t) stream;
    return GEIST_HIP_OK;
}

/* What the configuration asks for after the precedence rules. */
struct Resolved {
    bool  greedy;
    bool  use_k, use_p, use_m;
    int   k;
    float top_p, min_p, inv_t;
};

static int resolve(geist_hip_sampler *s, const struct geist_hip_sample_params *p, size_t n_vocab,
                   Resolved &r) {
    if (!p)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null params");
    const float T = p->temperature;
    r             = Resolved{};
    if (!(T > 0.0f)) { /* T == 0 in the dispatch, T < 0 inside each sampler: argmax, no draw */
        r.greedy = true;
        return GEIST_HIP_OK;
    }
    r.inv_t = 1.0f / T; /* sampler.c:77 */
    const bool p_set = p->top_p > 0.0f && p->top_p < 1.0f;
    if (p->precedence == GEIST_HIP_PRECEDENCE_REFERENCE) {
        if (p->min_p != 0.0f)
            return fail(s, GEIST_HIP_E_INVALID_ARG,
                        "min_p needs GEIST_HIP_PRECEDENCE_CHAIN (the reference has no min-p)");
        if (p->top_k > 1) { /* head.c:174-176: top-k wins, top_p is not consulted */
            r.use_k = (size_t) p->top_k < n_vocab; /* sampler.c:187-189 */
        } else if (p_set) {
            r.use_p = true;
        }
    } else if (p->precedence == GEIST_HIP_PRECEDENCE_CHAIN) {
        r.use_k = p->top_k > 1 && (size_t) p->top_k < n_vocab;
        r.use_p = p_set;
        r.use_m = p->min_p > 0.0f;
    } else {
        return fail(s, GEIST_HIP_E_INVALID_ARG, "unknown precedence %d", p->precedence);
    }
    r.k     = r.use_k ? (p->top_k > 8192 ? 8192 : p->top_k) : 0; /* sampler.c:213-215 */
    r.top_p = r.use_p ? p->top_p : 1.0f;
    r.min_p = r.use_m ? p->min_p : 0.0f;
    return GEIST_HIP_OK;
}

/* Everything that can make a sampling call fail on its arguments, without side effects: the
 * entry points that draw from a generator check first, so that a rejected call consumes no
 * draw. */
static int check_call(geist_hip_sampler *s, const struct geist_hip_rows *rows,
                      const struct geist_hip_sample_params *params, const void *d_out) {
    if (!rows || !params)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null rows or params");
    if (!d_out)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null output");
    Resolved rs;
    const int rc = resolve(s, params, rows->n_vocab, rs);
    if (rc)
        return rc;
    Launch L{};
    return make_launch(s, rows, params, !rs.greedy, L);
}

/* The meeting slots for a launch of rows * n_chunks workgroups (`words` per workgroup): this
 * launch takes the array whose turn it is, which the launch before left zero, and zeroes what
 * that launch used in the other. */
/* `one_xcd`: the launch deals the workgroups that meet to one XCD (rows in eights,
 * xcd_row_chunk); where the device was seen to place them so they meet through that XCD's L2
 * (MeetSpace::local). geist_hip_sampler_handoff_scope(s, 1) switches that off as well. */
static MeetSpace meet_space(geist_hip_sampler *s, const Launch &L, uint32_t words = 1,
                            bool one_xcd = false) {
    MeetState &st = *s->meet;
    if (st.suspect) { /* only after a failed launch: start again from two zeroed arrays */
        for (int t = 0; t < 2; ++t)
            launch_zero_words(s->stream, st.slots[t], st.capacity);
        st.used[0] = st.used[1] = 0;
        st.suspect              = false;
    }
    MeetSpace  m;
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (st.recorded && hipStreamIsCapturing(s->stream, &capture) == hipSuccess &&
        capture == hipStreamCaptureStatusActive) {
        /* being recorded: the launch meets in the array kept for graphs, and a fill kernel
         * recorded in front of it clears what it uses on every replay */
        const uint32_t n = words * (uint32_t) L.rows * (uint32_t) L.rv.n_chunks;
        launch_zero_words(s->stream, st.recorded, n);
        m.slots       = st.recorded;
        m.stale       = st.recorded;
        m.stale_count = 0;
        m.wait_limit  = s->wait_limit;
        m.local       = one_xcd && s->fused_wg_default != 0 && !s->handoff_far;
        return m;
    }
    m.slots       = st.slots[st.turn];
    m.stale       = st.slots[st.turn ^ 1];
    m.stale_count = st.used[st.turn ^ 1];
    m.wait_limit  = s->wait_limit;
    m.local       = one_xcd && s->fused_wg_default != 0 && !s->handoff_far;
    st.used[st.turn]     = words * (uint32_t) L.rows * (uint32_t) L.rv.n_chunks;
    st.used[st.turn ^ 1] = 0;
    st.turn ^= 1;
    return m;
}

static int sample_impl(geist_hip_sampler *s, const struct geist_hip_rows *rows,
                       const struct geist_hip_sample_params *params, const float *d_uniforms,
                       geist_hip_token_t *d_out) {
    if (s) {
        s->epoch_by_kernel = false;
        s->tell = false;
        if (s->notify && s->h_done) {
            /* (a launch recorded into a graph would report the same number at every replay:
             * recorded calls report nothing) */
            hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
            s->tell = hipStreamIsCapturing(s->stream, &capture) != hipSuccess ||
                      capture != hipStreamCaptureStatusActive;
        }
    }
    const int rc = gs_host::sample_stages(s, rows, params, d_uniforms, d_out, gs_host::STAGE_ALL, nullptr);
    if (rc == GEIST_HIP_OK && s->tell) {
        /* the ids of this call are written when the word holds this epoch */
        const Notify nt = {s->h_done, s->epoch + 1, s->rows_done};
        if (!s->epoch_by_kernel)
            launch_publish_epoch(s->stream, nt);
        s->epoch += 1;
    }
    return rc;
}

/* The buffers of the full-vocabulary top-p / min-p path (a row of probabilities per logit row
 * among them: hence not part of every sampler). All or nothing: a failure leaves no pointer set. */
static int reserve_sorted_workspace(geist_hip_sampler *s) {
    if (s->probs)
        return GEIST_HIP_OK;
    const size_t  R = s->max_rows;
    gs::CandSpace c = {};
    float        *probs = nullptr;
    hipError_t    e = hipSetDevice(s->device);
    if (e == hipSuccess) e = hipMalloc((void **) &c.row_bound, R * sizeof(int32_t));
    if (e == hipSuccess) e = hipMalloc((void **) &c.out_key, R * sizeof(uint32_t));
    if (e == hipSuccess) e = hipMalloc((void **) &c.key, R * CAND_CAP * sizeof(uint32_t));
    if (e == hipSuccess) e = hipMalloc((void **) &c.idx, R * CAND_CAP * sizeof(uint32_t));
    if (e == hipSuccess) e = hipMalloc((void **) &c.count, R * gs::CAND_COUNT_STRIDE * sizeof(int32_t));
    if (e == hipSuccess) e = hipMalloc((void **) &c.row_sum, R * sizeof(double));
    if (e == hipSuccess) e = hipMalloc((void **) &c.path, R * sizeof(int32_t));
    if (e == hipSuccess) e = hipMalloc((void **) &probs, R * s->max_vocab * sizeof(float));
    void     *walk_rows = nullptr;
    uint32_t *walk_hint = nullptr;
    if (e == hipSuccess) e = hipMalloc(&walk_rows, gs::walk_coop_bytes(R));
    if (e == hipSuccess) e = hipMemsetAsync(walk_rows, 0, gs::walk_coop_bytes(R), s->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(s->stream);
    if (e == hipSuccess) e = hipHostMalloc((void **) &walk_hint, 64, hipHostMallocDefault);
    if (e != hipSuccess) {
        void *ptrs[] = {c.row_bound, c.out_key, c.key, c.idx, c.count, c.row_sum, c.path, probs,
                        walk_rows};
        for (void *q : ptrs)
            if (q)
                (void) hipFree(q);
        if (walk_hint)
            (void) hipHostFree(walk_hint);
        return fail(s, e == hipErrorOutOfMemory ? GEIST_HIP_E_OOM : GEIST_HIP_E_BACKEND,
                    "workspace of the top-p / min-p path: %s", hipGetErrorString(e));
    }
    s->cand  = c;
    s->probs = probs;
    walk_hint[0] = walk_hint[1] = 0u;
    s->walk_rows = walk_rows;
    s->walk_hint = walk_hint;
    return GEIST_HIP_OK;
}

} /* extern "C" */

/* One sampling call is enqueued in up to three stages: a first pass over the rows where the mode
 * needs two (the row maxima before the exp-sum), the pass that streams the logits, and what
 * follows it per row. geist_hip_sample_rows runs both. */
int gs_host::sample_stages(geist_hip_sampler *s, const struct geist_hip_rows *rows,
                           const struct geist_hip_sample_params *params, const float *d_uniforms,
                           geist_hip_token_t *d_out, unsigned stages, const char **stream_kernel) {
    const bool do_stream = stages & gs_host::STAGE_STREAM,
               do_tail = stages & gs_host::STAGE_TAIL;
    const char *unused_name;
    if (!stream_kernel)
        stream_kernel = &unused_name;
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_out)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null output");
    Resolved rs;
    int      rc = resolve(s, params, rows ? rows->n_vocab : 0, rs);
    if (rc)
        return rc;
    Launch L;
    rc = make_launch(s, rows, params, !rs.greedy, L);
    if (rc)
        return rc;
    if (!rs.greedy && !d_uniforms)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "stochastic configuration without uniforms");
    HIPCHK(s, hipSetDevice(s->device));

    FinalLaunch f{};
    f.inv_t      = rs.inv_t;
    f.top_p      = rs.top_p;
    f.min_p      = rs.min_p;
    f.uniforms   = d_uniforms;
    f.chunk_best = s->chunk_best;
    f.chunk_sum  = s->chunk_sum;
    f.tmax       = s->tmax;
    f.out        = d_out;

    if (!rs.greedy && !rs.use_k && !(s->meet && s->meet->slots[0] && s->meet->slots[1]))
        return fail(s, GEIST_HIP_E_INTERNAL, "no meeting slots for the one-pass kernel");
    if (rs.greedy) {
        L.rv.stream_loads = s->logits_streamed;
        *stream_kernel    = "k_tmax_scan";
        if (do_stream)
            launch_tmax_scan(L, s->tmax, s->chunk_best);
        f.mode = FINAL_ARGMAX;
        if (do_tail)
            launch_row_final(L, f);
        return after_launch(s, "argmax");
    }
    if (rs.use_k) {
        if (rs.k > TOPK_FAST_MAX) {
            f.mode         = FINAL_TOPK;
            f.k            = rs.k;
            *stream_kernel = "k_topk_general";
            const int e    = do_stream ? launch_topk_general(L, f) : 0;
            if (e != 0)
                return fail(s, GEIST_HIP_E_BACKEND, "top-k (general) launch: %s",
                            hipGetErrorString((hipError_t) e));
            return after_launch(s, "top-k (general)");
        }
        /* the thread-maxima path wants the large chunks whatever the batch size: the final
         * kernel holds one key per scanning thread in LDS */
        L.nv           = 8;
        L.rv.per_chunk = 8192;
        L.rv.n_chunks  = (int) ((rows->n_vocab + 8191) / 8192);
        /* Penalties that can only lower a logit (rep >= 1, freq >= 0, pres >= 0) need not be
         * applied while scanning: the raw thread maxima then bound the penalised ones from
         * above, the final kernel penalises the elements it re-reads and checks that k of them
         * still reach the bound -- which proves that no element outside the re-read threads can
         * belong to the top k. A margin on the rank of the bound keeps that check from failing
         * when several leading logits are penalised away; a row that still fails takes the
         * general path. */
        Launch scan = L;
        f.k_sel     = rs.k;
        if (L.pen && L.rv.rep >= 1.0f && L.rv.freq >= 0.0f && L.rv.pres >= 0.0f) {
            scan.pen         = false;
            scan.rv.hist     = nullptr;
            scan.rv.hist_len = nullptr;
            const int margin = rs.k / 2 > 8 ? rs.k / 2 : 8;
            f.k_sel          = rs.k + margin < TOPK_FAST_MAX ? rs.k + margin : TOPK_FAST_MAX;
        }
        scan.rv.stream_loads = s->logits_streamed; /* the one pass over the rows */
        /* The soft-cap keeps the order of the logits, so the scan runs on the logits as they are
         * and the row-final kernel caps what it keeps (with the thread maxima already there from
         * a projection's epilogue they are uncapped as well). */
        f.cap_after = L.rv.softcap > 0.0f;
        if (f.cap_after)
            scan.rv.softcap = 0.0f;
        f.mode = FINAL_TOPK;
        f.k    = rs.k;
        /* Plain rows (aligned, no mask, penalties absent or left to the final kernel)
         * take the candidate path: the scan's wavefronts hand their leading groups on and the
         * row-final kernel gathers nothing. */
        const size_t row_waves = rows->rows * (size_t) L.rv.n_chunks * NWAVES_PER_CHUNK;
        const bool   plain = rs.k <= CAND_K_MAX && L.rv.vec_ok && !L.rv.allowed &&
                           L.rv.n_chunks <= CAND_CHUNKS_MAX && (!L.pen || !scan.pen) &&
                           !s->tmax_ready && s->wcands && row_waves <= s->wcands_row_waves;
        const int m = plain ? cand_lanes_for(f.k_sel, rows->n_vocab) : 0;
        /* a batch that fits the device in one round of 1024-thread workgroups takes scan and
         * row-final stage in one launch (the measuring stages cannot split it: the streaming
         * stage is the whole step) */
        /* a workgroup scans 32768 logits; launches of up to 128 workgroups halve that, so
         * that twice the compute units fetch a row (64 x 128256: 13.1 us with whole, 14.9 with
         * half workgroups; 32 rows 11.4 and 12.0; 16 rows 11.1 and 11.0; 4 rows 10.6 and 10.3;
         * one row 10.2 and 9.9, without penalties 9.0 and 8.6) */
        const size_t wgs_row8 = (size_t) ((L.rv.n_chunks + 3) / 4);
        const size_t wgs_row4 = (rows->n_vocab + 16383) / 16384;
        const bool   halves   = wgs_row4 <= (size_t) OL_WG_MAX && rows->rows * wgs_row4 <= 128;
        const size_t wgs_row = halves ? wgs_row4 : wgs_row8;
        const size_t wgs     = rows->rows * wgs_row;
        const bool   one     = plain && s->row_arrive &&
                             wgs <= (size_t) s->fused_wg_limit && rows->n_vocab % 4 == 0 &&
                             wg_cands_bytes(rows->rows, wgs_row) <= wave_cands_bytes(s->wcands_row_waves);
        const size_t per_wg  = halves ? 16384 : 32768;
        const size_t e_full  = rows->n_vocab < per_wg ? rows->n_vocab : per_wg;
        const int    r_full  = one ? cand_rank_for(f.k_sel, rows->n_vocab, e_full) : 0;
        const int    r_last  = one ? cand_rank_for(f.k_sel, rows->n_vocab,
                                                   rows->n_vocab - (wgs_row - 1) * per_wg) : 0;
        const int    r_w     = r_full && r_last ? r_full : 0;
        if (r_w) {
            f.row_flag         = s->row_flag; /* which path served each row, for diagnostics */
            s->topk_paths_rows = rows->rows;
            *stream_kernel     = "k_cand_scan_final";
            /* with both stages in this call, the kernel itself reports the ids written */
            Notify nt = {nullptr, 0, nullptr};
            if (s->tell && s->rows_done && do_stream && do_tail) {
                nt                 = Notify{s->h_done, s->epoch + 1, s->rows_done};
                s->epoch_by_kernel = true;
            }
            if (do_stream)
                launch_cand_scan_final(scan, L, f, s->tmax, wg_cands_at(s->wcands, rows->rows, wgs_row),
                                       r_w, r_last, reinterpret_cast<uint32_t *>(s->row_arrive),
                                       s->handoff_far, nt, (int) wgs_row, halves ? 4 : 8);
            return after_launch(s, "top-k");
        }
        if (m) {
            const WaveCands wc = wave_cands_at(s->wcands, row_waves);
            f.row_flag         = s->row_flag;
            s->topk_paths_rows = rows->rows;
            *stream_kernel     = "k_cand_scan";
            if (do_stream)
                launch_cand_scan(scan, s->tmax, wc, m);
            if (do_tail)
                launch_final_cand(L, f, wc);
            return after_launch(s, "top-k");
        }
        s->topk_paths_rows = 0;
        *stream_kernel     = "k_tmax_scan";
        if (!s->tmax_ready && do_stream)
            launch_tmax_scan(scan, s->tmax, nullptr);
        if (do_tail)
            launch_row_final(L, f);
        return after_launch(s, "top-k");
    }
    if (!rs.use_p && !rs.use_m) {
        Launch scan          = L;
        scan.rv.stream_loads = s->logits_streamed; /* the one pass over the rows */
        if (scan.nv == 2 && (size_t) scan.rows * (size_t) scan.rv.n_chunks <= 256) {
            /* A few rows: the step is a chain of waits, not of bytes, and a second launch is a
             * tenth of it. Scan, sums and the draw in one kernel (10.9 against 11.8 us for one
             * row of 128256, 12.0 against 12.7 for four; from 16 rows on the two kernels are the
             * faster form, their workgroups being smaller and gone sooner). The measuring
             * stages cannot split it: the streaming stage is the whole step. */
            *stream_kernel = "k_temperature_draw";
            if (do_stream)
                launch_temperature_draw(scan, rs.inv_t, d_uniforms, d_out,
                                        meet_space(s, scan, 2, true));
            return after_launch(s, "temperature");
        }
        *stream_kernel = "k_scan_expsum";
        if (do_stream &&
            launch_scan_expsum(scan, rs.inv_t, nullptr, s->chunk_best, s->chunk_sum, nullptr, 0,
                               nullptr, nullptr, 0, s->slab_sum,
                               meet_space(s, scan, 1, (scan.rows & 7) == 0), s->fast_sums))
            return fail(s, GEIST_HIP_E_BACKEND, "no launch geometry for the exp-sum pass");
        f.mode     = FINAL_TEMPERATURE;
        f.slab_sum = s->slab_sum;
        if (do_tail)
            launch_row_final(L, f);
        return after_launch(s, "temperature");
    }
    /* top-p and/or min-p over the whole vocabulary */
    rc = reserve_sorted_workspace(s); /* a no-op after geist_hip_sampler_prepare() or a first call */
    if (rc)
        return rc;
    L.nv           = 8;
    L.rv.per_chunk = 8192;
    L.rv.n_chunks  = (int) ((rows->n_vocab + 8191) / 8192);
    if (L.rv.n_chunks > s->max_chunks)
        return fail(s, GEIST_HIP_E_UNSUPPORTED, "n_vocab %zu needs more than %d chunks",
                    rows->n_vocab, s->max_chunks);
    /* min-p bounds the kept prefix by the row maximum alone, so the exp-sum pass can list the
     * candidates on its way; rows whose list overflows fall back to the bound of the row-final
     * kernel and a third pass */
    const int zb_m    = zbin_of_min_p(rs.min_p);
    f.cand            = s->cand;
    f.minp_listed     = rs.use_m && zb_m < ZBINS - 1;
    /* A min-p of a few percent keeps the list short on any plausible row, and the walk can follow
     * the exp-sum pass at once. Below that a flat row may overflow the list, and the row-final
     * kernel should get the chance to bound it by top-p instead. */
    f.minp_direct     = f.minp_listed && rs.min_p >= 0.02f;
    *stream_kernel = "k_scan_expsum";
    Launch scan          = L;
    scan.rv.stream_loads = s->logits_streamed; /* the one pass over whole rows */
    if (do_stream &&
        /* (the thread maxima are the row-final kernel's; with the list walk coming first and
         * alone nobody reads them) */
        launch_scan_expsum(scan, rs.inv_t, f.minp_direct ? nullptr : s->tmax, s->chunk_best,
                           s->chunk_sum, nullptr, 0, nullptr, f.minp_listed ? &f.cand : nullptr,
                           zb_m, nullptr, meet_space(s, scan, 1, (scan.rows & 7) == 0), s->fast_sums))
        return fail(s, GEIST_HIP_E_BACKEND, "no launch geometry for the exp-sum pass");
    if (!do_tail)
        return after_launch(s, "exp-sum scan");
    f.mode     = FINAL_SORTED;
    f.row_flag = s->row_flag;
    /* rows whose kept prefix is too wide for the shortcut of the row-final kernel flag themselves
     * 1: their candidates are listed and walked; what that cannot serve either takes the
     * whole-row walk inside the list-walk kernel. Each of these kernels returns at once for every
     * row not flagged for it. With the candidates already listed by the exp-sum pass the list
     * walk comes first and alone. */
    if (!f.minp_direct)
        launch_row_final(L, f);
    /* Rows that neither shortcut nor list can serve are walked in full: by their one workgroup
     * inside the list-walk kernel, or spread over the workgroups of their chunks by a kernel
     * behind it. That kernel is a launch more for every call, so it is sent only while such rows
     * keep turning up: the kernels say so in a page-locked word, which is looked at here without
     * waiting for anything (a stale value costs time, never a token). */
    WalkCoop wc = {};
    wc.rows       = s->walk_rows;
    wc.hint       = s->walk_hint;
    wc.wait_limit = s->wait_limit;
    if (s->walk_rows && s->walk_hint) {
        /* (calls are numbered from 1; a hint from one of the last 64 calls counts: with
         * several calls in flight the kernels' word lags behind) */
        const uint32_t call   = ++s->walk_calls;
        const uint32_t walked = __atomic_load_n(&s->walk_hint[0], __ATOMIC_RELAXED);
        const uint32_t ranout = __atomic_load_n(&s->walk_hint[1], __ATOMIC_RELAXED);
        wc.call   = call;
        /* the spread form holds two workgroups per compute unit: beyond a few rounds of them the
         * rows' own workgroups, all at once, are the faster way */
        const bool fits = rows->rows * (size_t) L.rv.n_chunks <= 1280;
        wc.spread = s->walk_mode == GEIST_HIP_WHOLE_ROW_WALK_SPREAD ||
                    (s->walk_mode == GEIST_HIP_WHOLE_ROW_WALK_ADAPTIVE && fits && walked != 0u &&
                     call - walked <= 64u);
        if (wc.spread) {
            wc.clear = (ranout != 0u && (int32_t) (ranout - s->walk_cleared) >= 0) ||
                       s->walk_clear;
            if (wc.clear)
                s->walk_cleared = call;
            s->walk_clear = s->wait_limit < 1024u; /* (a bound set for tests: clear behind it) */
            wc.step_base  = s->walk_steps;
            s->walk_steps += 16u;
        }
    }
    launch_candidates(L, f, s->probs, (long) s->max_vocab, wc);
    return after_launch(s, "top-p / min-p");
}

extern "C" {

int geist_hip_sample_rows(geist_hip_sampler *s, const struct geist_hip_rows *rows,
                          const struct geist_hip_sample_params *params, const float *d_uniforms,
                          geist_hip_token_t *d_out_tokens) {
    return sample_impl(s, rows, params, d_uniforms, d_out_tokens);
}

int geist_hip_sampler_set_wait_limit(geist_hip_sampler *s, uint32_t polls) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    s->wait_limit = polls;
    return GEIST_HIP_OK;
}

int geist_hip_sampler_one_launch_topk(geist_hip_sampler *s, int enable) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    s->fused_wg_limit = enable ? s->fused_wg_default : 0;
    return s->fused_wg_limit > 0 ? 1 : 0;
}

int geist_hip_sampler_set_whole_row_walk(geist_hip_sampler *s, int mode) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (mode != GEIST_HIP_WHOLE_ROW_WALK_ADAPTIVE && mode != GEIST_HIP_WHOLE_ROW_WALK_SPREAD &&
        mode != GEIST_HIP_WHOLE_ROW_WALK_ONE_WORKGROUP)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "unknown whole-row walk mode %d", mode);
    s->walk_mode = mode;
    return GEIST_HIP_OK;
}

int geist_hip_sampler_handoff_scope(geist_hip_sampler *s, int always_agent) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    s->handoff_far = always_agent != 0;
    return GEIST_HIP_OK;
}

int geist_hip_sampler_notify_ids(geist_hip_sampler *s, int enable) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (enable && !s->h_done) {
        HIPCHK(s, hipSetDevice(s->device));
        uint64_t *h = nullptr;
        uint32_t *d = nullptr;
        hipError_t e = hipHostMalloc((void **) &h, 64, hipHostMallocDefault);
        if (e == hipSuccess) e = hipMalloc((void **) &d, 64);
        if (e == hipSuccess) e = hipMemsetAsync(d, 0, 64, s->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(s->stream);
        if (e != hipSuccess) {
            if (h) (void) hipHostFree(h);
            if (d) (void) hipFree(d);
            return fail(s, e == hipErrorOutOfMemory ? GEIST_HIP_E_OOM : GEIST_HIP_E_BACKEND,
                        "the word that reports written ids: %s", hipGetErrorString(e));
        }
        *h           = 0;
        s->h_done    = h;
        s->rows_done = d;
    }
    s->notify = enable != 0;
    return GEIST_HIP_OK;
}

int geist_hip_sampler_wait_ids(geist_hip_sampler *s) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (s->notify && s->h_done && s->epoch != 0) {
        const volatile uint64_t *w = s->h_done;
        struct timespec t0, t1;
        clock_gettime(CLOCK_MONOTONIC, &t0);
        for (;;) {
            for (int i = 0; i < 256; ++i) {
                if (*w >= s->epoch) {
                    __atomic_thread_fence(__ATOMIC_ACQUIRE);
                    return GEIST_HIP_OK;
                }
                __builtin_ia32_pause();
            }
            clock_gettime(CLOCK_MONOTONIC, &t1);
            const double us = (double) (t1.tv_sec - t0.tv_sec) * 1e6 + (double) (t1.tv_nsec - t0.tv_nsec) * 1e-3;
            if (us > (double) s->wait_spin_us)
                break;
        }
    }
    /* not told within the time (or telling is off): wait for the stream, which also reports a
     * failed launch or kernel */
    return geist_hip_sampler_sync(s);
}

int geist_hip_sampler_set_wait_spin(geist_hip_sampler *s, uint32_t microseconds) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    s->wait_spin_us = microseconds;
    return GEIST_HIP_OK;
}

int geist_hip_sampler_set_sums(geist_hip_sampler *s, int mode) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (mode != GEIST_HIP_SUMS_EXACT && mode != GEIST_HIP_SUMS_FAST)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "sums: GEIST_HIP_SUMS_EXACT or GEIST_HIP_SUMS_FAST");
    s->fast_sums = mode == GEIST_HIP_SUMS_FAST;
    return GEIST_HIP_OK;
}

int geist_hip_sampler_one_launch_spec(geist_hip_sampler *s, int enable) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    s->spec_one_launch = enable != 0;
    return s->spec_one_launch ? 1 : 0;
}

int geist_hip_sampler_prepare(geist_hip_sampler *s, const struct geist_hip_sample_params *params,
                              size_t n_vocab) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    Resolved rs;
    int      rc = resolve(s, params, n_vocab ? n_vocab : s->max_vocab, rs);
    if (rc)
        return rc;
    if (!rs.greedy && !rs.use_k && (rs.use_p || rs.use_m))
        rc = reserve_sorted_workspace(s);
    return rc;
}

int geist_hip_sample_rows_static(int device, void *stream, const struct geist_hip_rows *rows,
                                 const struct geist_hip_sample_params *params,
                                 const float *d_uniforms, geist_hip_token_t *d_out_tokens,
                                 char *err, size_t err_len) {
    if (err && err_len)
        err[0] = 0;
    if (!rows || !params)
        return report(err, err_len, GEIST_HIP_E_INVALID_ARG, "null rows or params");
    /* a sampler object on the stack whose workspace is the device array: the flows below are
     * those of geist_hip_sample_rows, with the modes that need more than this left out */
    geist_hip_sampler tmp;
    tmp.device = device;
    tmp.stream = (hipStream_t) stream;
    Resolved rs;
    int      rc = resolve(&tmp, params, rows->n_vocab, rs);
    if (rc)
        return report(err, err_len, rc, "%s", tmp.err);
    if (!rs.greedy && !rs.use_k && (rs.use_p || rs.use_m))
        return report(err, err_len, GEIST_HIP_E_UNSUPPORTED,
                      "top-p / min-p over the whole vocabulary needs a row of probabilities per "
                      "logit row: use geist_hip_sample_rows");
    const size_t units = rows->rows * ((rows->n_vocab + 2047) / 2048);
    if (rows->rows == 0 || rows->n_vocab == 0 || units > STATIC_UNITS)
        return report(err, err_len, GEIST_HIP_E_INVALID_ARG,
                      "rows x ceil(n_vocab / 2048) = %zu x %zu exceeds the static workspace of %zu "
                      "(or the batch is empty)",
                      rows->rows, (rows->n_vocab + 2047) / 2048, (size_t) STATIC_UNITS);
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess)
        return report(err, err_len, GEIST_HIP_E_BACKEND, "hipSetDevice(%d): %s", device, hipGetErrorString(e));
    unsigned char *ws = nullptr;
    e                 = static_workspace(device, &ws);
    if (e != hipSuccess || !ws)
        return report(err, err_len, GEIST_HIP_E_BACKEND, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    tmp.max_rows   = rows->rows;
    tmp.max_vocab  = rows->n_vocab;
    tmp.max_chunks = (int) std::min<size_t>((rows->n_vocab + 2047) / 2048, (size_t) MAX_CHUNKS);
    tmp.tmax       = reinterpret_cast<float *>(ws + STATIC_TMAX);
    tmp.chunk_best = reinterpret_cast<uint64_t *>(ws + STATIC_BEST);
    tmp.chunk_sum  = reinterpret_cast<double *>(ws + STATIC_CSUM);
    tmp.slab_sum   = reinterpret_cast<double *>(ws + STATIC_SLAB);
    tmp.wcands     = ws + STATIC_WCANDS;
    tmp.wcands_row_waves = STATIC_ROW_WAVES;
    MeetState &ms = g_static_meet[device];
    ms.slots[0]   = reinterpret_cast<uint64_t *>(ws + STATIC_MEET);
    ms.slots[1]   = ms.slots[0] + 2 * STATIC_UNITS;
    ms.recorded   = ms.slots[1] + 2 * STATIC_UNITS;
    ms.capacity   = (uint32_t) (2 * STATIC_UNITS);
    tmp.meet      = &ms;
    rc = sample_impl(&tmp, rows, params, d_uniforms, d_out_tokens);
    return rc ? report(err, err_len, rc, "%s", tmp.err) : GEIST_HIP_OK;
}

int geist_hip_sample_rows_rng(geist_hip_sampler *s, const struct geist_hip_rows *rows,
                              const struct geist_hip_sample_params *params,
                              uint64_t *d_rng_states, int shared,
                              geist_hip_token_t *d_out_tokens) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!rows || !params)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null rows or params");
    const int rc = check_call(s, rows, params, d_out_tokens);
    if (rc)
        return rc;
    const bool greedy = !(params->temperature > 0.0f);
    if (!greedy) {
        if (!d_rng_states)
            return fail(s, GEIST_HIP_E_INVALID_ARG, "null rng states");
        HIPCHK(s, hipSetDevice(s->device));
        launch_rng_units(s->stream, d_rng_states, shared, (int) rows->rows, s->uniforms);
    }
    return sample_impl(s, rows, params, greedy ? nullptr : s->uniforms, d_out_tokens);
}

int geist_hip_argmax_f32(geist_hip_sampler *s, const float *d_logits, size_t n,
                         int32_t *out_index) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!out_index)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null out_index");
    struct geist_hip_rows r{};
    r.d_logits = d_logits;
    r.ld       = n;
    r.rows     = 1;
    r.n_vocab  = n;
    struct geist_hip_sample_params p{};
    p.repetition_penalty = 1.0f;
    int rc = sample_impl(s, &r, &p, nullptr, s->scalar_out);
    if (rc)
        return rc;
    HIPCHK(s, hipMemcpyAsync(s->h_scalar, s->scalar_out, sizeof(int32_t), hipMemcpyDeviceToHost,
                             s->stream));
    HIPCHK(s, hipStreamSynchronize(s->stream));
    *out_index = s->h_scalar[0];
    return GEIST_HIP_OK;
}

int geist_hip_apply_penalties(geist_hip_sampler *s, float *d_logits, size_t ld, size_t rows,
                              size_t n_vocab, const int32_t *d_history, size_t history_ld,
                              const int32_t *d_history_len, float rep, float freq, float pres) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_history || !d_history_len)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null history");
    struct geist_hip_rows r{};
    r.d_logits      = d_logits;
    r.ld            = ld;
    r.rows          = rows;
    r.n_vocab       = n_vocab;
    r.d_history     = d_history;
    r.history_ld    = history_ld;
    r.d_history_len = d_history_len;
    struct geist_hip_sample_params p{};
    p.repetition_penalty = rep;
    p.frequency_penalty  = freq;
    p.presence_penalty   = pres;
    Launch L;
    int    rc = make_launch(s, &r, &p, false, L);
    if (rc)
        return rc;
    if (!L.pen)
        return GEIST_HIP_OK; /* neutral parameters: nothing to do */
    HIPCHK(s, hipSetDevice(s->device));
    launch_penalties(L, d_logits);
    return after_launch(s, "penalties");
}

int geist_hip_softmax_rows(geist_hip_sampler *s, const struct geist_hip_rows *rows,
                           const struct geist_hip_sample_params *params, float *d_probs,
                           size_t ld_probs) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!params || !d_probs)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null params or output");
    if (!(params->temperature > 0.0f))
        return fail(s, GEIST_HIP_E_INVALID_ARG, "softmax needs temperature > 0");
    Launch L;
    int    rc = make_launch(s, rows, params, true, L);
    if (rc)
        return rc;
    if (ld_probs < rows->n_vocab)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "ld_probs < n_vocab");
    const float inv_t = 1.0f / params->temperature;
    HIPCHK(s, hipSetDevice(s->device));
    if (launch_scan_expsum(L, inv_t, nullptr, s->chunk_best, s->chunk_sum, nullptr, 0, nullptr,
                           nullptr, 0, nullptr, meet_space(s, L, 1, (L.rows & 7) == 0), s->fast_sums))
        return fail(s, GEIST_HIP_E_BACKEND, "no launch geometry for the exp-sum pass");
    launch_write_probs(L, inv_t, s->chunk_best, s->chunk_sum, d_probs, (long) ld_probs, nullptr);
    return after_launch(s, "softmax");
}

int geist_hip_logprob_rows(geist_hip_sampler *s, const float *d_logits, size_t ld, size_t rows,
                           size_t n_vocab, float logit_softcap, const int32_t *d_tokens,
                           size_t tokens_ld, size_t k_per_row, double *d_out, size_t out_ld) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_tokens || !d_out)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null tokens or output");
    if (k_per_row == 0 || tokens_ld < k_per_row || out_ld < k_per_row)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "k_per_row %zu with strides %zu / %zu", k_per_row,
                    tokens_ld, out_ld);
    if (k_per_row > 0x7fffffffu)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "k_per_row too large");
    struct geist_hip_rows          r = {d_logits, ld, rows, n_vocab, nullptr, 0, nullptr};
    struct geist_hip_sample_params p = {};
    p.temperature        = 1.0f;
    p.repetition_penalty = 1.0f;
    p.logit_softcap      = logit_softcap;
    Launch L;
    int    rc = make_launch(s, &r, &p, true, L);
    if (rc)
        return rc;
    HIPCHK(s, hipSetDevice(s->device));
    launch_tmax_scan(L, s->tmax, s->chunk_best);
    launch_logprob(L, s->chunk_best, s->chunk_sum, d_tokens, (long) tokens_ld, (int) k_per_row,
                   d_out, (long) out_ld);
    return after_launch(s, "log-probabilities");
}

int geist_hip_rmsnorm_rows(geist_hip_sampler *s, const float *d_x, size_t ld_x,
                           const float *d_weight, float eps, size_t n_rows, size_t n, float *d_y,
                           size_t ld_y) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_x || !d_weight || !d_y)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (n_rows == 0 || n == 0 || n > 0x7fffffffu || n_rows > 0x7fffffffu || ld_x < n || ld_y < n)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "rmsnorm: %zu rows of %zu, strides %zu / %zu",
                    n_rows, n, ld_x, ld_y);
    HIPCHK(s, hipSetDevice(s->device));
    launch_rmsnorm_rows(s->stream, d_x, (long) ld_x, d_weight, eps, (int) n_rows, (int) n, d_y,
                        (long) ld_y);
    return after_launch(s, "rmsnorm");
}

int geist_hip_f16_gemv_rows(geist_hip_sampler *s, const uint16_t *d_w_f16, size_t n_out,
                            size_t n_in, const float *d_x, size_t ld_x, size_t n_rows, float *d_y,
                            size_t ld_y) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_w_f16 || !d_x || !d_y)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (n_out == 0 || n_in == 0 || n_rows == 0 || n_in > 0x7ffffff8u || ld_x < n_in ||
        ld_y < n_out)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "gemv: %zu x %zu, %zu rows, strides %zu / %zu",
                    n_out, n_in, n_rows, ld_x, ld_y);
    if (n_in % 8 != 0)
        return fail(s, GEIST_HIP_E_UNSUPPORTED, "gemv: n_in %zu is not a multiple of 8", n_in);
    if (((uintptr_t) d_w_f16) % 16 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "gemv: weights not 16-byte aligned");
    HIPCHK(s, hipSetDevice(s->device));
    for (size_t m0 = 0; m0 < n_rows; m0 += GEMV_M_MAX) {
        const size_t m = n_rows - m0 < (size_t) GEMV_M_MAX ? n_rows - m0 : (size_t) GEMV_M_MAX;
        launch_f16_gemv(s->stream, d_w_f16, (long) n_out, (int) n_in, d_x + m0 * ld_x, (long) ld_x,
                        (int) m, d_y + m0 * ld_y, (long) ld_y);
    }
    return after_launch(s, "f16 gemv");
}

/* Scratch of the f64 projection: activations in double, their stage norms, the list of outputs
 * for the second kernel. */
static int f64_scratch(geist_hip_sampler *s, size_t n_out, size_t n_in, F64Scratch &ws) {
    if (s->f64_in < n_in || s->f64_out < n_out) {
        if (s->f64_ws) {
            HIPCHK(s, hipStreamSynchronize(s->stream));
            (void) hipFree(s->f64_ws);
            s->f64_ws = nullptr, s->f64_in = s->f64_out = 0;
        }
        const size_t in = n_in > s->f64_in ? n_in : s->f64_in;
        const size_t out = n_out > s->f64_out ? n_out : s->f64_out;
        const size_t bytes = (size_t) F64_M_MAX * (in + in / 64 + 2) * sizeof(double) + 16 +
                             out * F64_M_MAX * sizeof(int2);
        if (hipMalloc(&s->f64_ws, bytes) != hipSuccess) {
            s->f64_ws = nullptr;
            return fail(s, GEIST_HIP_E_OOM, "f64 projection: scratch");
        }
        s->f64_in = in, s->f64_out = out;
    }
    char *p      = static_cast<char *>(s->f64_ws);
    ws.xd        = reinterpret_cast<double *>(p);
    ws.xs        = ws.xd + (size_t) F64_M_MAX * s->f64_in;
    ws.amb_count = reinterpret_cast<int *>(ws.xs + (size_t) F64_M_MAX * (s->f64_in / 64 + 2));
    ws.amb_list  = reinterpret_cast<int2 *>(reinterpret_cast<char *>(ws.amb_count) + 16);
    return GEIST_HIP_OK;
}

static int f16_linear_impl(geist_hip_sampler *s, const uint16_t *d_w_f16, size_t n_out, size_t n_in,
                           const float *d_x, size_t ld_x, size_t n_rows, float *d_y, size_t ld_y) {
    F64Scratch ws;
    const int  rc = f64_scratch(s, n_out, n_in, ws);
    if (rc)
        return rc;
    for (size_t m0 = 0; m0 < n_rows; m0 += F64_M_MAX) {
        const size_t m = n_rows - m0 < (size_t) F64_M_MAX ? n_rows - m0 : (size_t) F64_M_MAX;
        launch_f16_linear_f64(s->stream, d_w_f16, (long) n_out, (int) n_in, d_x + m0 * ld_x,
                              (long) ld_x, (int) m, ws, d_y + m0 * ld_y, (long) ld_y);
    }
    return GEIST_HIP_OK;
}

/* Scratch of the Q6_K projection: the activations in double, their sums and magnitudes per
 * group of 16, the list of outputs for the second kernel. */
/* the int8 activations of the x86 kernels: one row for the Q6_K decode kernel, Q6X_M_MAX rows
 * for its batch path, Q4X_M_MAX rows for Q4_K */
static size_t q8_act_bytes(size_t n_in) {
    const size_t q6 = (n_in / 256) * Q8K_ACT_DWORDS;
    const size_t q4 = (size_t) Q4X_M_MAX * ((n_in / 256) * Q4X_ACT_DWORDS + Q4X_ACT_TAIL);
    const size_t qb = (size_t) Q6X_M_MAX * q6k_x86_batch_act_dwords((int) n_in);
    return (q6 > q4 ? (q6 > qb ? q6 : qb) : (q4 > qb ? q4 : qb)) * sizeof(uint32_t);
}

static int q6k_scratch(geist_hip_sampler *s, size_t n_out, size_t n_in, Q6KScratch &ws) {
    if (s->q6k_in < n_in || s->q6k_out < n_out) {
        if (s->q6k_ws) {
            HIPCHK(s, hipStreamSynchronize(s->stream));
            (void) hipFree(s->q6k_ws);
            s->q6k_ws = nullptr, s->q6k_in = s->q6k_out = 0;
        }
        const size_t in = n_in > s->q6k_in ? n_in : s->q6k_in;
        const size_t out = n_out > s->q6k_out ? n_out : s->q6k_out;
        const size_t bytes = (size_t) Q6K_M_MAX * (in + in / 8) * sizeof(double) + 16 +
                             out * Q6K_M_MAX * sizeof(int2) +
                             q8_act_bytes(in);
        if (hipMalloc(&s->q6k_ws, bytes) != hipSuccess) {
            s->q6k_ws = nullptr;
            return fail(s, GEIST_HIP_E_OOM, "Q6_K projection: scratch");
        }
        s->q6k_in = in, s->q6k_out = out;
    }
    char *p      = static_cast<char *>(s->q6k_ws);
    ws.xd        = reinterpret_cast<double *>(p);
    ws.xsum      = ws.xd + (size_t) Q6K_M_MAX * s->q6k_in;
    ws.xabs      = ws.xsum + (size_t) Q6K_M_MAX * (s->q6k_in / 16);
    ws.amb_count = reinterpret_cast<int *>(ws.xabs + (size_t) Q6K_M_MAX * (s->q6k_in / 16));
    ws.amb_list  = reinterpret_cast<int2 *>(reinterpret_cast<char *>(ws.amb_count) + 16);
    ws.act8      = reinterpret_cast<uint32_t *>(ws.amb_list + s->q6k_out * Q6K_M_MAX);
    return GEIST_HIP_OK;
}

static int q6k_linear_impl(geist_hip_sampler *s, const void *d_w_q6k, size_t n_out, size_t n_in,
                           const float *d_x, size_t ld_x, size_t n_rows, float *d_y, size_t ld_y) {
    Q6KScratch ws;
    const int  rc = q6k_scratch(s, n_out, n_in, ws);
    if (rc)
        return rc;
    for (size_t m0 = 0; m0 < n_rows; m0 += Q6K_M_MAX) {
        const size_t m = n_rows - m0 < (size_t) Q6K_M_MAX ? n_rows - m0 : (size_t) Q6K_M_MAX;
        launch_q6k_linear(s->stream, static_cast<const uint8_t *>(d_w_q6k), (long) n_out,
                          (int) n_in, d_x + m0 * ld_x, (long) ld_x, (int) m, ws, d_y + m0 * ld_y,
                          (long) ld_y);
    }
    return GEIST_HIP_OK;
}

static int q6k_packed_linear_impl(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                  size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                  float *d_y, size_t ld_y) {
    Q6KScratch ws;
    const int  rc = q6k_scratch(s, n_out, n_in, ws);
    if (rc)
        return rc;
    for (size_t m0 = 0; m0 < n_rows; m0 += Q6K_M_MAX) {
        const size_t m = n_rows - m0 < (size_t) Q6K_M_MAX ? n_rows - m0 : (size_t) Q6K_M_MAX;
        launch_q6k_packed_linear(s->stream, d_packed, (long) n_out, (int) n_in, d_x + m0 * ld_x,
                                 (long) ld_x, (int) m, ws, d_y + m0 * ld_y, (long) ld_y);
    }
    return GEIST_HIP_OK;
}

/* The x86 backend's decode kernel, row by row (each row is a pass over the table, as each call
 * of q6k_gemv_m1 is). */
static int q6k_gemv_x86_impl(geist_hip_sampler *s, const void *d_table, bool packed, size_t n_out,
                            size_t n_in, const float *d_x, size_t ld_x, size_t n_rows, float *d_y,
                            size_t ld_y) {
    Q6KScratch ws;
    const int  rc = q6k_scratch(s, n_out, n_in, ws);
    if (rc)
        return rc;
    for (size_t m = 0; m < n_rows; ++m) {
        launch_q8k_quantize(s->stream, d_x + m * ld_x, (long) ld_x, 1, (int) n_in, ws.act8);
        if (packed)
            launch_q6k_packed_gemv_q8k(s->stream, d_table, (long) n_out, (int) n_in, ws.act8,
                                       d_y + m * ld_y);
        else
            launch_q6k_gemv_q8k(s->stream, static_cast<const uint8_t *>(d_table), (long) n_out,
                                (int) n_in, ws.act8, d_y + m * ld_y);
    }
    return GEIST_HIP_OK;
}

/* cpu_x86_linear_q6k_mN (linear_q6k.c:234-300) over the packed copy or the table as it lies,
 * Q6X_M_MAX rows per pass over the table; one row is cpu_x86_linear_q6k_m1's decode kernel. The lane kernels' arithmetic for
 * tables of a multiple of 8 rows unless the host reproduced has no AVX-512 VNNI. */
static int q6k_x86_batch_impl(geist_hip_sampler *s, const void *d_table, bool packed, size_t n_out,
                              size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                              float *d_y, size_t ld_y) {
    if (n_rows == 1)
        return q6k_gemv_x86_impl(s, d_table, packed, n_out, n_in, d_x, ld_x, 1, d_y, ld_y);
    Q6KScratch ws;
    const int  rc = q6k_scratch(s, n_out, n_in, ws);
    if (rc)
        return rc;
    const bool lanes = !s->projection_avx2 && n_out % 8 == 0;
    for (size_t m0 = 0; m0 < n_rows; m0 += Q6X_M_MAX) {
        const size_t m = n_rows - m0 < (size_t) Q6X_M_MAX ? n_rows - m0 : (size_t) Q6X_M_MAX;
        launch_q8s_row_quantize(s->stream, d_x + m0 * ld_x, (long) ld_x, (int) m, (int) n_in,
                                ws.act8);
        launch_q6k_gemm_q8s(s->stream, d_table, packed, (long) n_out, (int) n_in, ws.act8, (int) m,
                            lanes, d_y + m0 * ld_y, (long) ld_y);
    }
    return GEIST_HIP_OK;
}

static int q6k_check(geist_hip_sampler *s, const void *d_w_q6k, size_t n_out, size_t n_in) {
    if (n_out == 0 || n_in == 0 || n_in > 0x7fffff00u || n_out > 0x7fffffffu)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "Q6_K table: %zu x %zu", n_out, n_in);
    if (n_in % 256 != 0)
        return fail(s, GEIST_HIP_E_UNSUPPORTED,
                    "Q6_K table: n_in %zu is not a multiple of the 256-element block", n_in);
    if (((uintptr_t) d_w_q6k) % 4 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "Q6_K table not 4-byte aligned");
    return GEIST_HIP_OK;
}

int geist_hip_q6k_linear_reserve(geist_hip_sampler *s, size_t n_out, size_t n_in) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    const int rc = q6k_check(s, nullptr, n_out, n_in);
    if (rc)
        return rc;
    HIPCHK(s, hipSetDevice(s->device));
    Q6KScratch ws;
    return q6k_scratch(s, n_out, n_in, ws);
}

int geist_hip_q6k_linear_rows(geist_hip_sampler *s, const void *d_w_q6k, size_t n_out, size_t n_in,
                              const float *d_x, size_t ld_x, size_t n_rows, float *d_y,
                              size_t ld_y) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_w_q6k || !d_x || !d_y)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (n_rows == 0 || ld_x < n_in || ld_y < n_out)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "Q6_K linear: %zu rows, strides %zu / %zu", n_rows,
                    ld_x, ld_y);
    int rc = q6k_check(s, d_w_q6k, n_out, n_in);
    if (rc)
        return rc;
    HIPCHK(s, hipSetDevice(s->device));
    rc = q6k_linear_impl(s, d_w_q6k, n_out, n_in, d_x, ld_x, n_rows, d_y, ld_y);
    return rc ? rc : after_launch(s, "Q6_K linear");
}

size_t geist_hip_q6k_packed_bytes(size_t n_out, size_t n_in) {
    if (n_out == 0 || n_in == 0 || n_in % 256 != 0 || n_in > 0x7fffff00u || n_out > 0x7fffffffu)
        return 0;
    return q6k_packed_bytes((long) n_out, (int) n_in);
}

int geist_hip_q6k_pack(geist_hip_sampler *s, const void *d_w_q6k, size_t n_out, size_t n_in,
                       void *d_packed) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_w_q6k || !d_packed)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    const int rc = q6k_check(s, d_w_q6k, n_out, n_in);
    if (rc)
        return rc;
    if (((uintptr_t) d_packed) % 16 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "packed Q6_K table not 16-byte aligned");
    HIPCHK(s, hipSetDevice(s->device));
    launch_q6k_pack(s->stream, static_cast<const uint8_t *>(d_w_q6k), (long) n_out, (int) n_in,
                    d_packed);
    return after_launch(s, "Q6_K pack");
}

int geist_hip_q6k_packed_linear_rows(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                     size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                     float *d_y, size_t ld_y) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_packed || !d_x || !d_y)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (n_rows == 0 || ld_x < n_in || ld_y < n_out)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "Q6_K linear: %zu rows, strides %zu / %zu", n_rows,
                    ld_x, ld_y);
    int rc = q6k_check(s, d_packed, n_out, n_in);
    if (rc)
        return rc;
    if (((uintptr_t) d_packed) % 16 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "packed Q6_K table not 16-byte aligned");
    HIPCHK(s, hipSetDevice(s->device));
    rc = q6k_packed_linear_impl(s, d_packed, n_out, n_in, d_x, ld_x, n_rows, d_y, ld_y);
    return rc ? rc : after_launch(s, "Q6_K linear (packed)");
}

int geist_hip_q6k_packed_gemv_x86_rows(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                       size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                       float *d_y, size_t ld_y) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_packed || !d_x || !d_y)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (n_rows == 0 || ld_x < n_in || ld_y < n_out)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "Q6_K decode: %zu rows, strides %zu / %zu", n_rows,
                    ld_x, ld_y);
    int rc = q6k_check(s, d_packed, n_out, n_in);
    if (rc)
        return rc;
    if (((uintptr_t) d_packed) % 16 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "packed Q6_K table not 16-byte aligned");
    HIPCHK(s, hipSetDevice(s->device));
    rc = q6k_gemv_x86_impl(s, d_packed, true, n_out, n_in, d_x, ld_x, n_rows, d_y, ld_y);
    return rc ? rc : after_launch(s, "Q6_K decode (packed)");
}

int geist_hip_q6k_packed_linear_x86_rows(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                         size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                         float *d_y, size_t ld_y) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_packed || !d_x || !d_y)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (n_rows == 0 || ld_x < n_in || ld_y < n_out)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "Q6_K x86 batch: %zu rows, strides %zu / %zu",
                    n_rows, ld_x, ld_y);
    int rc = q6k_check(s, d_packed, n_out, n_in);
    if (rc)
        return rc;
    if (((uintptr_t) d_packed) % 16 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "packed Q6_K table not 16-byte aligned");
    HIPCHK(s, hipSetDevice(s->device));
    rc = q6k_x86_batch_impl(s, d_packed, true, n_out, n_in, d_x, ld_x, n_rows, d_y, ld_y);
    return rc ? rc : after_launch(s, "Q6_K x86 batch (packed)");
}

int geist_hip_q6k_linear_x86_rows(geist_hip_sampler *s, const void *d_w_q6k, size_t n_out,
                                  size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                  float *d_y, size_t ld_y) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_w_q6k || !d_x || !d_y)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (n_rows == 0 || ld_x < n_in || ld_y < n_out)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "Q6_K x86 batch: %zu rows, strides %zu / %zu",
                    n_rows, ld_x, ld_y);
    int rc = q6k_check(s, d_w_q6k, n_out, n_in);
    if (rc)
        return rc;
    HIPCHK(s, hipSetDevice(s->device));
    rc = q6k_x86_batch_impl(s, d_w_q6k, false, n_out, n_in, d_x, ld_x, n_rows, d_y, ld_y);
    return rc ? rc : after_launch(s, "Q6_K x86 batch");
}

int geist_hip_q6k_gemv_x86_rows(geist_hip_sampler *s, const void *d_w_q6k, size_t n_out,
                                size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                float *d_y, size_t ld_y) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_w_q6k || !d_x || !d_y)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (n_rows == 0 || ld_x < n_in || ld_y < n_out)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "Q6_K decode: %zu rows, strides %zu / %zu", n_rows,
                    ld_x, ld_y);
    int rc = q6k_check(s, d_w_q6k, n_out, n_in);
    if (rc)
        return rc;
    HIPCHK(s, hipSetDevice(s->device));
    rc = q6k_gemv_x86_impl(s, d_w_q6k, false, n_out, n_in, d_x, ld_x, n_rows, d_y, ld_y);
    return rc ? rc : after_launch(s, "Q6_K decode");
}

size_t geist_hip_q8k_act_bytes(size_t n_in, size_t n_rows) {
    if (n_in == 0 || n_in % 256 != 0 || n_in > 0x7fffff00u)
        return 0;
    return n_rows * (n_in / 256) * Q8K_ACT_DWORDS * sizeof(uint32_t);
}

int geist_hip_q8k_quantize_rows(geist_hip_sampler *s, const float *d_x, size_t ld_x, size_t n_rows,
                                size_t n_in, void *d_act) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_x || !d_act)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (n_rows == 0 || n_rows > 65535 || n_in == 0 || n_in > 0x7fffff00u || ld_x < n_in)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "int8 activations: %zu rows of %zu, stride %zu",
                    n_rows, n_in, ld_x);
    if (n_in % 256 != 0)
        return fail(s, GEIST_HIP_E_UNSUPPORTED, "int8 activations: %zu is not a multiple of 256",
                    n_in);
    if (((uintptr_t) d_act) % 64 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "int8 activations: buffer not 64-byte aligned");
    HIPCHK(s, hipSetDevice(s->device));
    launch_q8k_quantize(s->stream, d_x, (long) ld_x, (int) n_rows, (int) n_in,
                        static_cast<uint32_t *>(d_act));
    return after_launch(s, "int8 activations");
}

int geist_hip_q6k_packed_gemv_q8k(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                  size_t n_in, const void *d_act, float *d_y) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_packed || !d_act || !d_y)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    const int rc = q6k_check(s, d_packed, n_out, n_in);
    if (rc)
        return rc;
    if (((uintptr_t) d_packed) % 16 != 0 || ((uintptr_t) d_act) % 64 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "Q6_K decode: table or activations misaligned");
    HIPCHK(s, hipSetDevice(s->device));
    launch_q6k_packed_gemv_q8k(s->stream, d_packed, (long) n_out, (int) n_in,
                               static_cast<const uint32_t *>(d_act), d_y);
    return after_launch(s, "Q6_K decode (packed)");
}

static int q4k_packed_linear_impl(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                  size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                  float *d_y, size_t ld_y) {
    Q6KScratch ws; /* the activations in double: the Q6_K projection's scratch */
    const int  rc = q6k_scratch(s, n_out, n_in, ws);
    if (rc)
        return rc;
    for (size_t m0 = 0; m0 < n_rows; m0 += Q6K_M_MAX) {
        const size_t m = n_rows - m0 < (size_t) Q6K_M_MAX ? n_rows - m0 : (size_t) Q6K_M_MAX;
        launch_q4k_packed_linear(s->stream, d_packed, (long) n_out, (int) n_in, d_x + m0 * ld_x,
                                 (long) ld_x, (int) m, ws, d_y + m0 * ld_y, (long) ld_y);
    }
    return GEIST_HIP_OK;
}

/* Shapes the reference's x86 decode kernel takes (q4kx8_gemv_m1: rows in eights, at most 64
 * super-blocks per row); others go through other kernels of that backend, not reproduced. */
static bool q4k_x86_shape(size_t n_out, size_t n_in) {
    return n_out % 8 == 0 && n_in % 256 == 0 && n_in / 256 >= 1 && n_in / 256 <= 64;
}

/* batch: the rows are one call of cpu_x86_linear_q4k_mN (linear_q4k.c:198-250) -- a row count
 * that is a multiple of 4 takes the batch quantiser, a multiple of 16 over 16 n table rows the
 * arithmetic of the AVX-512 tiles unless the host reproduced has none; otherwise every row is a
 * call of the decode kernel. Q4X_M_MAX rows share a pass over the table. */
static int q4k_packed_x86_impl(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                               size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                               float *d_y, size_t ld_y, bool batch) {
    Q6KScratch ws;
    const int  rc = q6k_scratch(s, n_out, n_in, ws);
    if (rc)
        return rc;
    const bool kx4   = batch && n_rows > 1 && n_rows % 4 == 0;
    const bool pairs = kx4 && !s->projection_avx2 && n_rows % 16 == 0 && n_out % 16 == 0;
    const size_t tile = Q4X_M_MAX;
    for (size_t m0 = 0; m0 < n_rows; m0 += tile) {
        const size_t m = n_rows - m0 < tile ? n_rows - m0 : tile;
        launch_q8k_row_quantize(s->stream, d_x + m0 * ld_x, (long) ld_x, (int) m, (int) n_in, kx4,
                                ws.act8);
        launch_q4k_packed_gemv_q8k(s->stream, d_packed, (long) n_out, (int) n_in, ws.act8, (int) m,
                                   pairs, d_y + m0 * ld_y, (long) ld_y);
    }
    return GEIST_HIP_OK;
}

static int q4k_packed_x86_rows(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                               size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                               float *d_y, size_t ld_y, bool batch) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_packed || !d_x || !d_y)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (n_rows == 0 || ld_x < n_in || ld_y < n_out)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "Q4_K x86 kernels: %zu rows, strides %zu / %zu",
                    n_rows, ld_x, ld_y);
    int rc = q6k_check(s, d_packed, n_out, n_in);
    if (rc)
        return rc;
    if (!q4k_x86_shape(n_out, n_in))
        return fail(s, GEIST_HIP_E_UNSUPPORTED,
                    "Q4_K x86 kernels: %zu x %zu is not a shape they take (rows in eights, at "
                    "most 64 super-blocks per row)", n_out, n_in);
    if (((uintptr_t) d_packed) % 16 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "packed Q4_K table not 16-byte aligned");
    HIPCHK(s, hipSetDevice(s->device));
    rc = q4k_packed_x86_impl(s, d_packed, n_out, n_in, d_x, ld_x, n_rows, d_y, ld_y, batch);
    return rc ? rc : after_launch(s, "Q4_K x86 kernels (packed)");
}

int geist_hip_q4k_packed_gemv_x86_rows(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                       size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                       float *d_y, size_t ld_y) {
    return q4k_packed_x86_rows(s, d_packed, n_out, n_in, d_x, ld_x, n_rows, d_y, ld_y, false);
}

int geist_hip_q4k_packed_linear_x86_rows(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                         size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                         float *d_y, size_t ld_y) {
    return q4k_packed_x86_rows(s, d_packed, n_out, n_in, d_x, ld_x, n_rows, d_y, ld_y, true);
}

size_t geist_hip_q8k_row_act_bytes(size_t n_in) {
    if (n_in == 0 || n_in % 256 != 0 || n_in > 0x7fffff00u)
        return 0;
    return q4k_x86_act_dwords((int) n_in) * sizeof(uint32_t);
}

int geist_hip_q8k_row_quantize(geist_hip_sampler *s, const float *d_x, size_t n_in, void *d_act) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_x || !d_act)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (n_in == 0 || n_in > 0x7fffff00u)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "int8 activation row of %zu", n_in);
    if (n_in % 256 != 0)
        return fail(s, GEIST_HIP_E_UNSUPPORTED, "int8 activation row: %zu is not a multiple of 256",
                    n_in);
    if (((uintptr_t) d_act) % 64 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "int8 activation row: buffer not 64-byte aligned");
    HIPCHK(s, hipSetDevice(s->device));
    launch_q8k_row_quantize(s->stream, d_x, (long) n_in, 1, (int) n_in, false,
                            static_cast<uint32_t *>(d_act));
    return after_launch(s, "int8 activation row");
}

int geist_hip_q4k_packed_gemv_q8k(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                  size_t n_in, const void *d_act, float *d_y) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_packed || !d_act || !d_y)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    const int rc = q6k_check(s, d_packed, n_out, n_in);
    if (rc)
        return rc;
    if (!q4k_x86_shape(n_out, n_in))
        return fail(s, GEIST_HIP_E_UNSUPPORTED,
                    "Q4_K decode: %zu x %zu is not a shape of the x86 kernel (rows in eights, at "
                    "most 64 super-blocks per row)", n_out, n_in);
    if (((uintptr_t) d_packed) % 16 != 0 || ((uintptr_t) d_act) % 64 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "Q4_K decode: table or activations misaligned");
    HIPCHK(s, hipSetDevice(s->device));
    launch_q4k_packed_gemv_q8k(s->stream, d_packed, (long) n_out, (int) n_in,
                               static_cast<const uint32_t *>(d_act), 1, false, d_y, (long) n_out);
    return after_launch(s, "Q4_K decode (packed)");
}

size_t geist_hip_q4k_packed_bytes(size_t n_out, size_t n_in) {
    if (n_out == 0 || n_in == 0 || n_in % 256 != 0 || n_in > 0x7fffff00u)
        return 0;
    return q4k_packed_bytes((long) n_out, (int) n_in);
}

int geist_hip_q4k_pack(geist_hip_sampler *s, const void *d_w_q4k, size_t n_out, size_t n_in,
                       void *d_packed) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_w_q4k || !d_packed)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    const int rc = q6k_check(s, d_w_q4k, n_out, n_in); /* the same shape rules */
    if (rc)
        return rc;
    if (((uintptr_t) d_packed) % 16 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "packed Q4_K table not 16-byte aligned");
    HIPCHK(s, hipSetDevice(s->device));
    launch_q4k_pack(s->stream, static_cast<const uint8_t *>(d_w_q4k), (long) n_out, (int) n_in,
                    d_packed);
    return after_launch(s, "Q4_K pack");
}

int geist_hip_q4k_packed_linear_rows(geist_hip_sampler *s, const void *d_packed, size_t n_out,
                                     size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                                     float *d_y, size_t ld_y) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_packed || !d_x || !d_y)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (n_rows == 0 || ld_x < n_in || ld_y < n_out)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "Q4_K linear: %zu rows, strides %zu / %zu", n_rows,
                    ld_x, ld_y);
    int rc = q6k_check(s, d_packed, n_out, n_in);
    if (rc)
        return rc;
    if (((uintptr_t) d_packed) % 16 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "packed Q4_K table not 16-byte aligned");
    HIPCHK(s, hipSetDevice(s->device));
    rc = q4k_packed_linear_impl(s, d_packed, n_out, n_in, d_x, ld_x, n_rows, d_y, ld_y);
    return rc ? rc : after_launch(s, "Q4_K linear (packed)");
}

int geist_hip_f16_linear_reserve(geist_hip_sampler *s, size_t n_out, size_t n_in) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (n_out == 0 || n_in == 0 || n_in > 0x7ffffff8u)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "linear: %zu x %zu", n_out, n_in);
    HIPCHK(s, hipSetDevice(s->device));
    F64Scratch ws;
    return f64_scratch(s, n_out, n_in, ws);
}

int geist_hip_f16_linear_rows(geist_hip_sampler *s, const uint16_t *d_w_f16, size_t n_out,
                              size_t n_in, const float *d_x, size_t ld_x, size_t n_rows,
                              float *d_y, size_t ld_y) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_w_f16 || !d_x || !d_y)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (n_out == 0 || n_in == 0 || n_rows == 0 || n_in > 0x7ffffff8u || ld_x < n_in ||
        ld_y < n_out)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "linear: %zu x %zu, %zu rows, strides %zu / %zu",
                    n_out, n_in, n_rows, ld_x, ld_y);
    if (n_in % 8 != 0)
        return fail(s, GEIST_HIP_E_UNSUPPORTED, "linear: n_in %zu is not a multiple of 8", n_in);
    if (((uintptr_t) d_w_f16) % 16 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "linear: weights not 16-byte aligned");
    HIPCHK(s, hipSetDevice(s->device));
    const int rc = f16_linear_impl(s, d_w_f16, n_out, n_in, d_x, ld_x, n_rows, d_y, ld_y);
    return rc ? rc : after_launch(s, "f16 linear");
}

int geist_hip_f16_to_q8w(geist_hip_sampler *s, const uint16_t *d_w_f16, size_t n_out, size_t n_in,
                         int8_t *d_wq, float *d_scales) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_w_f16 || !d_wq || !d_scales || n_out == 0 || n_in == 0 || n_in > 0x7fffffffu ||
        n_out > 0x7fffffffu)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "f16_to_q8w: null argument or bad shape");
    HIPCHK(s, hipSetDevice(s->device));
    launch_f16_to_q8w(s->stream, d_w_f16, (long) n_out, (int) n_in, d_wq, d_scales);
    return after_launch(s, "f16_to_q8w");
}

int geist_hip_q8w_gemv_rows(geist_hip_sampler *s, const int8_t *d_wq, const float *d_scales,
                            size_t n_out, size_t n_in, const float *d_x, size_t ld_x,
                            size_t n_rows, float *d_y, size_t ld_y) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_wq || !d_scales || !d_x || !d_y)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (n_out == 0 || n_in == 0 || n_rows == 0 || n_in > 0x7ffffff0u || ld_x < n_in ||
        ld_y < n_out)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "q8w gemv: %zu x %zu, %zu rows, strides %zu / %zu",
                    n_out, n_in, n_rows, ld_x, ld_y);
    if (n_in % 16 != 0)
        return fail(s, GEIST_HIP_E_UNSUPPORTED, "q8w gemv: n_in %zu is not a multiple of 16", n_in);
    if (((uintptr_t) d_wq) % 16 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "q8w gemv: weights not 16-byte aligned");
    HIPCHK(s, hipSetDevice(s->device));
    for (size_t m0 = 0; m0 < n_rows; m0 += GEMV_M_MAX) {
        const size_t m = n_rows - m0 < (size_t) GEMV_M_MAX ? n_rows - m0 : (size_t) GEMV_M_MAX;
        launch_q8w_gemv(s->stream, d_wq, d_scales, (long) n_out, (int) n_in, d_x + m0 * ld_x,
                        (long) ld_x, (int) m, d_y + m0 * ld_y, (long) ld_y);
    }
    return after_launch(s, "q8w gemv");
}

/* Norm, projection and sampling; the table is binary16, int8 with one scale per row (d_scales),
 * or Q6_K super-blocks. */
enum { TABLE_F16 = 0, TABLE_Q8W = 1, TABLE_Q6K = 2, TABLE_Q6K_PACKED = 3, TABLE_Q4K_PACKED = 4 };
static int project_sample_impl(geist_hip_sampler *s, const float *d_hidden, size_t ld_hidden,
                               size_t rows, size_t d_model, const float *d_norm_weight,
                               float rms_eps, int table, const void *d_embed,
                               const float *d_scales, size_t n_vocab, float *d_normed,
                               float *d_logits, size_t ld_logits,
                               const struct geist_hip_sample_params *params,
                               const float *d_uniforms, uint64_t *d_rng_states, int shared,
                               geist_hip_token_t *d_out_tokens) {
    const bool      q8          = table == TABLE_Q8W;
    const bool      q6k         = table == TABLE_Q6K || table == TABLE_Q6K_PACKED ||
                                  table == TABLE_Q4K_PACKED; /* the block formats */
    const size_t    in_multiple = q6k ? 256 : q8 ? 16 : 8;
    const uint16_t *d_embed_f16 = (const uint16_t *) d_embed;
    const int8_t   *d_embed_q8  = (const int8_t *) d_embed;
    if (!d_hidden || !d_norm_weight || !d_embed || !d_logits || !params || !d_out_tokens)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (rows == 0 || rows > s->max_rows || d_model == 0 || d_model > 0x7ffffff8u ||
        n_vocab == 0 || n_vocab > s->max_vocab || ld_hidden < d_model || ld_logits < n_vocab)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "projection: %zu rows, d_model %zu, vocab %zu",
                    rows, d_model, n_vocab);
    if (d_model % in_multiple != 0)
        return fail(s, GEIST_HIP_E_UNSUPPORTED, "projection: d_model %zu is not a multiple of %zu",
                    d_model, in_multiple);
    if (((uintptr_t) d_embed) % 16 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "projection: weights not 16-byte aligned");
    Resolved rs;
    int      rc = resolve(s, params, n_vocab, rs);
    if (rc)
        return rc;
    if (!rs.greedy && !d_uniforms && !d_rng_states)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "stochastic configuration without draws");
    const struct geist_hip_rows r = {d_logits, ld_logits, rows, n_vocab, nullptr, 0, nullptr,
                                     nullptr, 0};
    if ((rc = check_call(s, &r, params, d_out_tokens)) != GEIST_HIP_OK)
        return rc; /* before any draw */
    HIPCHK(s, hipSetDevice(s->device));
    const bool f64     = table == TABLE_F16 && (rows > 1 || s->projection_portable);
    const bool fuse_ok = f16_gemv_can_fuse((int) rows) && !f64 && !q6k;
    /* the top-k path's scan is the projection's epilogue (its thread maxima are those of the
     * logits before the soft-cap, which the row-final kernel applies to what it keeps) */
    const bool topk_scan = fuse_ok && !rs.greedy && rs.use_k && rs.k <= TOPK_FAST_MAX;
    if (!d_normed)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "no buffer for the normed rows");
    /* one row over a Q6_K table on the x86 backend: its integer decode kernel
     * (q6k_gemv_m1), whose activation quantiser rides on the norm's launch */
    const bool q6k_x86 = (table == TABLE_Q6K_PACKED || table == TABLE_Q6K) && rows == 1 &&
                         !s->projection_portable;
    /* ... and over a packed Q4_K table of a shape that backend's kernels take: one row likewise
     * (q4kx8_gemv_m1), a batch as cpu_x86_linear_q4k_mN projects it */
    const bool q4k_x86  = table == TABLE_Q4K_PACKED && !s->projection_portable &&
                          q4k_x86_shape(n_vocab, d_model);
    const bool q4k_kx4   = q4k_x86 && rows > 1 && rows % 4 == 0;
    /* a batch over a Q6_K table as cpu_x86_linear_q6k_mN projects it */
    const bool q6k_x86_mn    = (table == TABLE_Q6K_PACKED || table == TABLE_Q6K) && rows > 1 &&
                               !s->projection_portable;
    const bool q6k_mn_fused  = q6k_x86_mn && rows <= (size_t) Q6X_M_MAX;
    const bool q4k_fused = q4k_x86 && rows <= (size_t) Q4X_M_MAX;
    Q6KScratch q6ws{};
    if (q6k_x86 || q4k_fused || q6k_mn_fused) {
        if ((rc = q6k_scratch(s, n_vocab, d_model, q6ws)) != GEIST_HIP_OK)
            return rc;
        if (q6k_x86)
            launch_rmsnorm_q8k_rows(s->stream, d_hidden, (long) ld_hidden, d_norm_weight, rms_eps,
                                    1, (int) d_model, d_normed, (long) d_model, q6ws.act8);
        else if (q6k_mn_fused)
            launch_rmsnorm_q8s_rows(s->stream, d_hidden, (long) ld_hidden, d_norm_weight, rms_eps,
                                    (int) rows, (int) d_model, d_normed, (long) d_model, q6ws.act8);
        else
            launch_rmsnorm_q8k_row_rows(s->stream, d_hidden, (long) ld_hidden, d_norm_weight,
                                        rms_eps, (int) rows, (int) d_model, d_normed,
                                        (long) d_model, q4k_kx4, q6ws.act8);
    } else {
        launch_rmsnorm_rows(s->stream, d_hidden, (long) ld_hidden, d_norm_weight, rms_eps,
                            (int) rows, (int) d_model, d_normed, (long) d_model);
    }
    if (topk_scan) {
        GemvFuse f{};
        f.tmax     = s->tmax;
        f.n_chunks = (int) ((n_vocab + 8191) / 8192);
        if (q8)
            launch_q8w_gemv(s->stream, d_embed_q8, d_scales, (long) n_vocab, (int) d_model,
                            d_normed, (long) d_model, (int) rows, d_logits, (long) ld_logits, &f);
        else
            launch_f16_gemv(s->stream, d_embed_f16, (long) n_vocab, (int) d_model, d_normed,
                            (long) d_model, (int) rows, d_logits, (long) ld_logits, &f);
    } else if (q6k_x86) {
        if (table == TABLE_Q6K_PACKED)
            launch_q6k_packed_gemv_q8k(s->stream, d_embed, (long) n_vocab, (int) d_model, q6ws.act8,
                                       d_logits);
        else
            launch_q6k_gemv_q8k(s->stream, static_cast<const uint8_t *>(d_embed), (long) n_vocab,
                                (int) d_model, q6ws.act8, d_logits);
    } else if (q6k_mn_fused) {
        launch_q6k_gemm_q8s(s->stream, d_embed, table == TABLE_Q6K_PACKED, (long) n_vocab,
                            (int) d_model, q6ws.act8, (int) rows,
                            !s->projection_avx2 && n_vocab % 8 == 0, d_logits, (long) ld_logits);
    } else if (q6k_x86_mn) {
        if ((rc = q6k_x86_batch_impl(s, d_embed, table == TABLE_Q6K_PACKED, n_vocab, d_model,
                                     d_normed, d_model, rows, d_logits, ld_logits)) != GEIST_HIP_OK)
            return rc;
    } else if (q4k_fused) {
        /* (at most 8 rows: never the AVX-512 tiles' arithmetic) */
        launch_q4k_packed_gemv_q8k(s->stream, d_embed, (long) n_vocab, (int) d_model, q6ws.act8,
                                   (int) rows, false, d_logits, (long) ld_logits);
    } else if (q4k_x86) {
        if ((rc = q4k_packed_x86_impl(s, d_embed, n_vocab, d_model, d_normed, d_model, rows,
                                      d_logits, ld_logits, true)) != GEIST_HIP_OK)
            return rc;
    } else if (q6k) {
        /* the portable kernel after dequant_q6_K_row, for one row and for a batch */
        rc = table == TABLE_Q4K_PACKED
                 ? q4k_packed_linear_impl(s, d_embed, n_vocab, d_model, d_normed, d_model, rows,
                                          d_logits, ld_logits)
             : table == TABLE_Q6K_PACKED
                 ? q6k_packed_linear_impl(s, d_embed, n_vocab, d_model, d_normed, d_model, rows,
                                          d_logits, ld_logits)
                 : q6k_linear_impl(s, d_embed, n_vocab, d_model, d_normed, d_model, rows, d_logits,
                                   ld_logits);
        if (rc)
            return rc;
    } else if (f64) {
        /* more than one row: the reference's batch kernel (cpu_scalar_w_quant_mN), its x86
         * kernels being decode-only; or the portable backend asked for */
        rc = f16_linear_impl(s, d_embed_f16, n_vocab, d_model, d_normed, d_model, rows, d_logits,
                             ld_logits);
        if (rc)
            return rc;
    } else {
        for (size_t m0 = 0; m0 < rows; m0 += GEMV_M_MAX) {
            const size_t m = rows - m0 < (size_t) GEMV_M_MAX ? rows - m0 : (size_t) GEMV_M_MAX;
            if (q8)
                launch_q8w_gemv(s->stream, d_embed_q8, d_scales, (long) n_vocab, (int) d_model,
                                d_normed + m0 * d_model, (long) d_model, (int) m,
                                d_logits + m0 * ld_logits, (long) ld_logits);
            else
                launch_f16_gemv(s->stream, d_embed_f16, (long) n_vocab, (int) d_model,
                                d_normed + m0 * d_model, (long) d_model, (int) m,
                                d_logits + m0 * ld_logits, (long) ld_logits);
        }
    }
    if (!rs.greedy && d_rng_states) {
        launch_rng_units(s->stream, d_rng_states, shared, (int) rows, s->uniforms);
        d_uniforms = s->uniforms;
    }
    s->tmax_ready = topk_scan;
    rc            = sample_impl(s, &r, params, rs.greedy ? nullptr : d_uniforms, d_out_tokens);
    s->tmax_ready = false;
    return rc;
}

int geist_hip_project_sample_rows(geist_hip_sampler *s, const float *d_hidden, size_t ld_hidden,
                                  size_t rows, size_t d_model, const float *d_norm_weight,
                                  float rms_eps, const uint16_t *d_embed_f16, size_t n_vocab,
                                  float *d_normed, float *d_logits, size_t ld_logits,
                                  const struct geist_hip_sample_params *params,
                                  const float *d_uniforms, uint64_t *d_rng_states, int shared,
                                  geist_hip_token_t *d_out_tokens) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    return project_sample_impl(s, d_hidden, ld_hidden, rows, d_model, d_norm_weight, rms_eps,
                               TABLE_F16, d_embed_f16, nullptr, n_vocab, d_normed, d_logits, ld_logits,
                               params, d_uniforms, d_rng_states, shared, d_out_tokens);
}

int geist_hip_project_sample_rows_q8w(geist_hip_sampler *s, const float *d_hidden,
                                      size_t ld_hidden, size_t rows, size_t d_model,
                                      const float *d_norm_weight, float rms_eps,
                                      const int8_t *d_embed_q8, const float *d_scales,
                                      size_t n_vocab, float *d_normed, float *d_logits,
                                      size_t ld_logits,
                                      const struct geist_hip_sample_params *params,
                                      const float *d_uniforms, uint64_t *d_rng_states, int shared,
                                      geist_hip_token_t *d_out_tokens) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_scales)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    return project_sample_impl(s, d_hidden, ld_hidden, rows, d_model, d_norm_weight, rms_eps,
                               TABLE_Q8W, d_embed_q8, d_scales, n_vocab, d_normed, d_logits, ld_logits,
                               params, d_uniforms, d_rng_states, shared, d_out_tokens);
}

int geist_hip_project_sample_rows_q6k(geist_hip_sampler *s, const float *d_hidden,
                                      size_t ld_hidden, size_t rows, size_t d_model,
                                      const float *d_norm_weight, float rms_eps,
                                      const void *d_embed_q6k, size_t n_vocab, float *d_normed,
                                      float *d_logits, size_t ld_logits,
                                      const struct geist_hip_sample_params *params,
                                      const float *d_uniforms, uint64_t *d_rng_states, int shared,
                                      geist_hip_token_t *d_out_tokens) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    return project_sample_impl(s, d_hidden, ld_hidden, rows, d_model, d_norm_weight, rms_eps,
                               TABLE_Q6K, d_embed_q6k, nullptr, n_vocab, d_normed, d_logits,
                               ld_logits, params, d_uniforms, d_rng_states, shared, d_out_tokens);
}

int geist_hip_project_sample_rows_q6k_packed(geist_hip_sampler *s, const float *d_hidden,
                                             size_t ld_hidden, size_t rows, size_t d_model,
                                             const float *d_norm_weight, float rms_eps,
                                             const void *d_embed_packed, size_t n_vocab,
                                             float *d_normed, float *d_logits, size_t ld_logits,
                                             const struct geist_hip_sample_params *params,
                                             const float *d_uniforms, uint64_t *d_rng_states,
                                             int shared, geist_hip_token_t *d_out_tokens) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    return project_sample_impl(s, d_hidden, ld_hidden, rows, d_model, d_norm_weight, rms_eps,
                               TABLE_Q6K_PACKED, d_embed_packed, nullptr, n_vocab, d_normed,
                               d_logits, ld_logits, params, d_uniforms, d_rng_states, shared,
                               d_out_tokens);
}

int geist_hip_project_sample_rows_q4k_packed(geist_hip_sampler *s, const float *d_hidden,
                                             size_t ld_hidden, size_t rows, size_t d_model,
                                             const float *d_norm_weight, float rms_eps,
                                             const void *d_embed_packed, size_t n_vocab,
                                             float *d_normed, float *d_logits, size_t ld_logits,
                                             const struct geist_hip_sample_params *params,
                                             const float *d_uniforms, uint64_t *d_rng_states,
                                             int shared, geist_hip_token_t *d_out_tokens) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    return project_sample_impl(s, d_hidden, ld_hidden, rows, d_model, d_norm_weight, rms_eps,
                               TABLE_Q4K_PACKED, d_embed_packed, nullptr, n_vocab, d_normed,
                               d_logits, ld_logits, params, d_uniforms, d_rng_states, shared,
                               d_out_tokens);
}

int geist_hip_propose_drafts_ngram(geist_hip_sampler *s, const int32_t *d_history,
                                   size_t history_ld, const int32_t *d_history_len,
                                   const geist_hip_token_t *d_seed, size_t n_seq, size_t k_max,
                                   size_t max_suffix, geist_hip_token_t *d_out_drafts,
                                   size_t out_ld, int32_t *d_out_count, int32_t *d_out_match_len) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_history || !d_history_len || !d_seed || !d_out_drafts || !d_out_count ||
        !d_out_match_len)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (n_seq == 0 || n_seq > 0x7fffffffu)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "n_seq %zu", n_seq);
    if (k_max == 0 || k_max > (size_t) NGRAM_DRAFT_MAX)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "k_max %zu (1..%d)", k_max, NGRAM_DRAFT_MAX);
    if (out_ld < k_max)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "out_ld %zu < k_max %zu", out_ld, k_max);
    HIPCHK(s, hipSetDevice(s->device));
    launch_ngram_draft(s->stream, d_history, (long) history_ld, d_history_len, d_seed, (int) n_seq,
                       (int) k_max, max_suffix > 64 ? 64 : (int) max_suffix, d_out_drafts,
                       (long) out_ld, d_out_count, d_out_match_len);
    return after_launch(s, "n-gram drafts");
}

int geist_hip_spec_verify(geist_hip_sampler *s, const float *d_target, size_t ld_t,
                          const float *d_draft_q, size_t ld_q, const int32_t *d_draft,
                          const float *d_uniforms, size_t n_seq, size_t L, size_t n_vocab,
                          float temperature, float logit_softcap,
                          geist_hip_token_t *d_out_tokens, int32_t *d_n_accepted) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_target || !d_draft || !d_out_tokens || !d_n_accepted)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (n_seq == 0 || L == 0 || L > (size_t) SPEC_DRAFT_MAX)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "n_seq %zu, draft length %zu (1..%d)", n_seq, L,
                    SPEC_DRAFT_MAX);
    const bool greedy = !(temperature > 0.0f);
    if (!greedy && !d_uniforms)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "stochastic verification needs uniforms");
    if (!greedy && d_draft_q && ld_q < n_vocab)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "ld_q < n_vocab");
    struct geist_hip_rows r{};
    r.d_logits = d_target;
    r.ld       = ld_t;
    r.rows     = n_seq * (L + 1);
    r.n_vocab  = n_vocab;
    struct geist_hip_sample_params p{};
    p.temperature        = temperature;
    p.repetition_penalty = 1.0f;
    p.logit_softcap      = logit_softcap;
    Launch La;
    int    rc = make_launch(s, &r, &p, !greedy, La); /* greedy rows skip the monotone cap */
    if (rc)
        return rc;
    HIPCHK(s, hipSetDevice(s->device));
    const float inv_t = greedy ? 1.0f : 1.0f / temperature;
    if (greedy)
        launch_tmax_scan(La, s->tmax, s->chunk_best);
    else {
        Launch scan          = La;
        scan.rv.stream_loads = s->logits_streamed; /* the one pass over whole rows */
        /* no slab sums: of the n_seq * (L + 1) rows at most n_seq are drawn from, each by a
         * workgroup that walks the located chunk from its start */
        if (launch_scan_expsum(scan, inv_t, nullptr, s->chunk_best, s->chunk_sum, d_draft, (int) L,
                               s->probe_p, nullptr, 0, nullptr,
                               meet_space(s, scan, 1, (scan.rows & 7) == 0), s->fast_sums))
            return fail(s, GEIST_HIP_E_BACKEND, "no launch geometry for the exp-sum pass");
    }
    SpecLaunch sp{};
    sp.n_seq      = (int) n_seq;
    sp.L          = (int) L;
    sp.greedy     = greedy ? 1 : 0;
    sp.inv_t      = inv_t;
    sp.q          = d_draft_q;
    sp.ld_q       = (long) ld_q;
    sp.draft      = d_draft;
    sp.uniforms   = d_uniforms;
    sp.chunk_best = s->chunk_best;
    sp.chunk_sum  = s->chunk_sum;
    sp.probe_p    = s->probe_p;
    sp.resid_sum  = s->resid_sum;
    sp.resid_slab = s->resid_slab;
    sp.slab_sum   = nullptr;
    sp.verdict    = s->verdict;
    sp.out_tokens = d_out_tokens;
    sp.n_accepted = d_n_accepted;
    /* the residual pass and the draw in one launch while its workgroups, at the two per compute
     * unit their registers allow, run in one round; past that the two kernels are the lighter */
    if (!greedy && s->spec_one_launch &&
        n_seq * (size_t) La.rv.n_chunks <= (size_t) gs::SPEC_ONE_LAUNCH_WGS_PER_CU * (size_t) s->cu_count) {
        Launch per_seq = La;
        per_seq.rows   = (int) n_seq;
        const MeetSpace m = meet_space(s, per_seq);
        launch_spec(La, sp, &m);
    } else {
        launch_spec(La, sp);
    }
    return after_launch(s, "spec verification");
}

/* ---- device-memory helpers ----------------------------------------------------------------- */
int geist_hip_malloc(geist_hip_sampler *s, size_t bytes, void **d_ptr) {
    if (!s || !d_ptr)
        return GEIST_HIP_E_INVALID_ARG;
    HIPCHK(s, hipSetDevice(s->device));
    HIPCHK(s, hipMalloc(d_ptr, bytes ? bytes : 1));
    return GEIST_HIP_OK;
}
int geist_hip_free(geist_hip_sampler *s, void *d_ptr) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    HIPCHK(s, hipFree(d_ptr));
    return GEIST_HIP_OK;
}
/* Page-locked host memory that the device addresses in place (hipHostMalloc: the pointer is valid
 * on both sides). What a kernel stores there is in host memory once its stream has been waited
 * for, and what the host stores there is what a kernel launched afterwards reads: a few words of
 * results or arguments cross without a copy command. */
int geist_hip_host_malloc(geist_hip_sampler *s, size_t bytes, void **h_ptr) {
    if (!s || !h_ptr)
        return GEIST_HIP_E_INVALID_ARG;
    HIPCHK(s, hipSetDevice(s->device));
    HIPCHK(s, hipHostMalloc(h_ptr, bytes ? bytes : 1, hipHostMallocDefault));
    return GEIST_HIP_OK;
}
int geist_hip_host_free(geist_hip_sampler *s, void *h_ptr) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (h_ptr)
        HIPCHK(s, hipHostFree(h_ptr));
    return GEIST_HIP_OK;
}
int geist_hip_upload(geist_hip_sampler *s, void *d_dst, const void *h_src, size_t bytes) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    HIPCHK(s, hipMemcpyAsync(d_dst, h_src, bytes, hipMemcpyHostToDevice, s->stream));
    HIPCHK(s, hipStreamSynchronize(s->stream));
    return GEIST_HIP_OK;
}
int geist_hip_download(geist_hip_sampler *s, void *h_dst, const void *d_src, size_t bytes) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    HIPCHK(s, hipMemcpyAsync(h_dst, d_src, bytes, hipMemcpyDeviceToHost, s->stream));
    HIPCHK(s, hipStreamSynchronize(s->stream));
    return GEIST_HIP_OK;
}

/* ---- speculative output head -------------------------------------------------------------- */

struct geist_hip_spec_head {
    gs::SpecHeadDev d      = {};
    int             device = 0;
};

int geist_hip_spec_head_geometry(size_t n_vocab, size_t d_model, size_t stride_override,
                                 size_t topk_override, size_t *sketch_dim, size_t *topk) {
    if (!sketch_dim || !topk || n_vocab == 0 || d_model == 0)
        return GEIST_HIP_E_INVALID_ARG;
    auto clamp = [](size_t v, size_t lo, size_t hi) { return v < lo ? lo : (v > hi ? hi : v); };
    /* spec_head.c:431-452 */
    const size_t stride_dflt = d_model > 640 ? d_model / 640 : 1;
    size_t       sub         = stride_override ? clamp(stride_override, 1, d_model) : stride_dflt;
    while (sub > 1 && d_model % sub != 0)
        sub--;
    const size_t k = topk_override ? clamp(topk_override, 16, n_vocab)
                                   : (n_vocab >= 200000 ? (size_t) 4096 : (size_t) 1024);
    if (n_vocab < 8192)
        return GEIST_HIP_E_UNSUPPORTED;
    const size_t sd = d_model / sub;
    if ((double) (2 * d_model) / (double) sd < 3.0)
        return GEIST_HIP_E_UNSUPPORTED;
    /* what the kernels take */
    if (sd % 16 != 0 || sd > (size_t) gs::SPEC_SKETCH_DIM_MAX || d_model % 16 != 0 ||
        d_model > (size_t) gs::SPEC_D_MODEL_MAX || k > n_vocab / 64 ||
        k > (size_t) gs::SPEC_TOPK_MAX || n_vocab > (size_t) gs::SPEC_VOCAB_MAX)
        return GEIST_HIP_E_UNSUPPORTED;
    *sketch_dim = sd;
    *topk       = k;
    return GEIST_HIP_OK;
}

void geist_hip_spec_head_destroy(geist_hip_sampler *s, geist_hip_spec_head *sh) {
    if (!sh)
        return;
    (void) s;
    (void) hipSetDevice(sh->device);
    gs::SpecHeadDev &d = sh->d;
    void *ptrs[] = {d.sketch, d.row_scale, d.w_drop, d.w_l1, d.dims, d.kept, d.act, d.rough,
                    d.gmax, d.sc, d.fin_idx, d.fin_exact};
    for (void *p : ptrs)
        if (p)
            (void) hipFree(p);
    delete sh;
}

int geist_hip_spec_head_build(geist_hip_sampler *s, const uint16_t *d_embed_f16, size_t n_vocab,
                              size_t d_model, size_t stride_override, size_t topk_override,
                              geist_hip_spec_head **out) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_embed_f16 || !out)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (((uintptr_t) d_embed_f16) % 16 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "sketch head: table not 16-byte aligned");
    size_t sd = 0, topk = 0;
    const int rc = geist_hip_spec_head_geometry(n_vocab, d_model, stride_override, topk_override,
                                                &sd, &topk);
    if (rc)
        return fail(s, rc, "sketch head: no sketch for vocab %zu, d_model %zu", n_vocab, d_model);
    HIPCHK(s, hipSetDevice(s->device));
    geist_hip_spec_head *sh = new (std::nothrow) geist_hip_spec_head;
    if (!sh)
        return fail(s, GEIST_HIP_E_OOM, "sketch head");
    sh->device         = s->device;
    gs::SpecHeadDev &d = sh->d;
    d.vocab = (long) n_vocab, d.d_model = (int) d_model, d.sketch_dim = (int) sd;
    d.topk = (int) topk, d.n_groups = (int) ((n_vocab + 31) / 32);
    d.list_cap = (int) (2 * topk);
    d.w        = d_embed_f16;
    float *d_var = nullptr;
    auto   alloc = [&](auto &p, size_t bytes) {
        return hipMalloc(reinterpret_cast<void **>(&p), bytes) == hipSuccess;
    };
    bool ok = alloc(d.sketch, n_vocab * sd) && alloc(d.row_scale, n_vocab * 4) &&
              alloc(d.w_drop, n_vocab * 4) && alloc(d.w_l1, n_vocab * 4) && alloc(d.dims, sd * 4) &&
              alloc(d.kept, d_model) && alloc(d.act, sd * 4) && alloc(d.rough, (size_t) ((n_vocab + 31) / 32) * 32 * 4) &&
              alloc(d.gmax, (size_t) d.n_groups * 4) && alloc(d.sc, sizeof(gs::SpecScalars)) &&
              alloc(d.fin_idx, topk * 4) && alloc(d.fin_exact, topk * 4) &&
              alloc(d_var, d_model * 4);
    int err = ok ? 0 : GEIST_HIP_E_OOM;
    std::vector<float>    var;
    std::vector<uint32_t> dims;
    std::vector<uint8_t>  kept;
    try { /* no exception leaves a C entry point */
        var.resize(d_model), dims.resize(sd), kept.assign(d_model, 0);
    } catch (const std::bad_alloc &) {
        err = GEIST_HIP_E_OOM;
    }
    if (!err) {
        /* spec_head.c:505-522 on the device, :526-548 here */
        const long vstep = n_vocab > 512 ? (long) (n_vocab / 512) : 1;
        gs::launch_spec_dim_stats(s->stream, d_embed_f16, (long) n_vocab, (int) d_model, vstep, d_var);
        if (hipMemcpyAsync(var.data(), d_var, d_model * 4, hipMemcpyDeviceToHost, s->stream) != hipSuccess ||
            hipStreamSynchronize(s->stream) != hipSuccess)
            err = GEIST_HIP_E_BACKEND;
    }
    if (!err) {
        for (size_t k = 0; k < sd; ++k) { /* the first of equals, as the reference's scan */
            size_t best = 0;
            for (size_t i = 1; i < d_model; ++i)
                if (var[i] > var[best])
                    best = i;
            dims[k]   = (uint32_t) best;
            var[best] = -1.0f;
        }
        std::sort(dims.begin(), dims.end());
        for (uint32_t i : dims)
            kept[i] = 1;
        if (hipMemcpyAsync(d.dims, dims.data(), sd * 4, hipMemcpyHostToDevice, s->stream) != hipSuccess ||
            hipMemcpyAsync(d.kept, kept.data(), d_model, hipMemcpyHostToDevice, s->stream) != hipSuccess)
            err = GEIST_HIP_E_BACKEND;
    }
    if (!err) {
        gs::launch_spec_sketch_rows(s->stream, d);
        if (hipGetLastError() != hipSuccess || hipStreamSynchronize(s->stream) != hipSuccess)
            err = GEIST_HIP_E_BACKEND;
    }
    if (d_var)
        (void) hipFree(d_var);
    if (err) {
        geist_hip_spec_head_destroy(s, sh);
        return fail(s, err, err == GEIST_HIP_E_OOM ? "sketch head: out of device memory"
                                                   : "sketch head: build failed");
    }
    *out = sh;
    return GEIST_HIP_OK;
}

int geist_hip_spec_head_view(const geist_hip_spec_head *sh, struct geist_hip_spec_head_view *out) {
    if (!sh || !out)
        return GEIST_HIP_E_INVALID_ARG;
    const gs::SpecHeadDev &d = sh->d;
    out->n_vocab = (size_t) d.vocab, out->d_model = (size_t) d.d_model;
    out->sketch_dim = (size_t) d.sketch_dim, out->topk = (size_t) d.topk;
    out->d_dims = d.dims, out->d_sketch = d.sketch, out->d_row_scale = d.row_scale;
    out->d_w_drop = d.w_drop, out->d_w_l1 = d.w_l1, out->d_rough = d.rough;
    return GEIST_HIP_OK;
}

int geist_hip_spec_head_try(geist_hip_sampler *s, geist_hip_spec_head *sh,
                            const float *d_hidden_normed, int verify,
                            struct geist_hip_spec_result *d_result) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!sh || !d_hidden_normed || !d_result)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (sh->device != s->device)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "sketch head built on another device");
    if (((uintptr_t) d_hidden_normed) % 16 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "sketch head: hidden row not 16-byte aligned");
    static_assert(sizeof(gs::SpecResult) == sizeof(struct geist_hip_spec_result), "result layout");
    HIPCHK(s, hipSetDevice(s->device));
    gs::launch_spec_try(s->stream, sh->d, d_hidden_normed, verify != 0,
                        reinterpret_cast<gs::SpecResult *>(d_result));
    return after_launch(s, "sketch head");
}

int geist_hip_spec_head_try_hidden(geist_hip_sampler *s, geist_hip_spec_head *sh,
                                   const float *d_hidden, const float *d_norm_weight,
                                   float rms_eps, float *d_normed, int verify,
                                   struct geist_hip_spec_result *d_result) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!sh || !d_hidden || !d_norm_weight || !d_normed || !d_result)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null argument");
    if (sh->device != s->device)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "sketch head built on another device");
    if (((uintptr_t) d_normed) % 16 != 0)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "sketch head: normed row not 16-byte aligned");
    HIPCHK(s, hipSetDevice(s->device));
    gs::launch_spec_try(s->stream, sh->d, d_hidden, verify != 0,
                        reinterpret_cast<gs::SpecResult *>(d_result), d_norm_weight, rms_eps,
                        d_normed);
    return after_launch(s, "sketch head");
}

int geist_hip_rng_draw_units(geist_hip_sampler *s, uint64_t *d_rng_state, size_t n,
                             float *d_out_units) {
    if (!s)
        return GEIST_HIP_E_INVALID_ARG;
    if (!d_rng_state || !d_out_units || n == 0 || n > 0x7fffffffu)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "null state or output, or n out of range");
    HIPCHK(s, hipSetDevice(s->device));
    launch_rng_units(s->stream, d_rng_state, /*shared=*/1, (int) n, d_out_units);
    return after_launch(s, "rng draws");
}

int geist_hip_sampler_topk_paths(geist_hip_sampler *s, int32_t *h_paths, size_t rows) {
    if (!s || !h_paths)
        return GEIST_HIP_E_INVALID_ARG;
    if (rows > s->max_rows)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "rows %zu > max_rows %zu", rows, s->max_rows);
    if (s->topk_paths_rows == 0 || rows > s->topk_paths_rows) {
        /* the last top-k call ran the thread-maxima path for every row (or there was none) */
        HIPCHK(s, hipStreamSynchronize(s->stream));
        for (size_t r = 0; r < rows; ++r)
            h_paths[r] = -1;
        return GEIST_HIP_OK;
    }
    return geist_hip_download(s, h_paths, s->row_flag, rows * sizeof(int32_t));
}

int geist_hip_sampler_row_paths(geist_hip_sampler *s, int32_t *h_paths, size_t rows) {
    if (!s || !h_paths)
        return GEIST_HIP_E_INVALID_ARG;
    if (rows > s->max_rows)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "rows %zu > max_rows %zu", rows, s->max_rows);
    if (!s->cand.path)
        return fail(s, GEIST_HIP_E_INVALID_ARG, "no full-vocabulary top-p / min-p call was made yet");
    return geist_hip_download(s, h_paths, s->cand.path, rows * sizeof(int32_t));
}

} /* extern "C" */
