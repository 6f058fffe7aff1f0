/*
 * sampler_dropin.c -- the symbols of the reference's src/engine/sampler.h on top of the HIP
 * path (C23). Each function keeps the reference's control flow around the sampling itself:
 * which configurations fall back to argmax, which consume a draw, and when
 * (src/engine/sampler.c:106-132, 178-228, 232-305). The arithmetic on the logits happens in
 * the kernels behind geist_sampler_hip.h.
 */
#include "geist_sampler_dropin.h"
#include "geist_sampler_hip.h"

#include <pthread.h>
#include <stdatomic.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* One device context per (thread, vocabulary size): the row buffer, the uniform and the result
 * slot. geist_sampler_argmax / _temperature have no workspace argument, so theirs is
 * thread-local, which keeps the reference's promise that all entry points are reentrant
 * (src/engine/sampler.h:8). */
struct dropin_ctx {
    geist_hip_sampler *hs;
    float             *d_row;
    float             *d_u;
    int32_t           *d_out;
    size_t             n_vocab;
};

#define DROPIN_MAGIC 0x4753414D504C5253ull /* "GSAMPLRS" */
struct ws_header {
    uint64_t          magic;
    struct dropin_ctx ctx;
    uint64_t          pad; /* keeps probs 16-byte aligned */
};

/* A device failure (no device, out of device memory, a failed copy or launch) goes to the failure
 * handler. The reference's samplers cannot fail (on a failed allocation they degrade to the
 * arg-max on the host, sampler.c:125-127); there is no host path here, so the default handler
 * ends the process with a message. A handler installed by the application may return instead:
 * the sampling call then returns GEIST_SAMPLER_DROPIN_FAILED_TOKEN. */
static _Atomic(geist_sampler_dropin_failure_fn) g_on_failure;
static _Atomic(void *)                          g_on_failure_user;

void geist_sampler_dropin_on_failure(geist_sampler_dropin_failure_fn fn, void *user) {
    atomic_store(&g_on_failure_user, user);
    atomic_store(&g_on_failure, fn);
}

static geist_token_t fail(const char *what, geist_hip_sampler *hs) {
    const char *detail = hs ? geist_hip_sampler_last_error(hs) : "no device context";
    const geist_sampler_dropin_failure_fn fn = atomic_load(&g_on_failure);
    if (fn != nullptr) {
        fn(what, detail, atomic_load(&g_on_failure_user));
        return GEIST_SAMPLER_DROPIN_FAILED_TOKEN;
    }
    fprintf(stderr, "geist sampler (HIP): %s: %s\n", what, detail);
    abort();
}

static void ctx_release(struct dropin_ctx *c) {
    if (c->hs != nullptr) {
        geist_hip_free(c->hs, c->d_row);
        geist_hip_host_free(c->hs, c->d_u);
        geist_hip_host_free(c->hs, c->d_out);
        geist_hip_sampler_destroy(c->hs);
    }
    *c = (struct dropin_ctx) {0};
}

static int ctx_setup(struct dropin_ctx *c, size_t n_vocab) {
    *c     = (struct dropin_ctx) {0};
    int rc = geist_hip_sampler_create(0, 1, n_vocab, nullptr, &c->hs);
    if (rc != GEIST_HIP_OK)
        return rc;
    void *p = nullptr;
    if ((rc = geist_hip_malloc(c->hs, n_vocab * sizeof(float), &p)) == GEIST_HIP_OK)
        c->d_row = p;
    /* the draw and the token id: page-locked host memory that the kernels read and write in
     * place, so neither is copied */
    if (rc == GEIST_HIP_OK &&
        (rc = geist_hip_host_malloc(c->hs, sizeof(float), &p)) == GEIST_HIP_OK)
        c->d_u = p;
    if (rc == GEIST_HIP_OK &&
        (rc = geist_hip_host_malloc(c->hs, sizeof(int32_t), &p)) == GEIST_HIP_OK)
        c->d_out = p;
    if (rc != GEIST_HIP_OK) {
        ctx_release(c);
        return rc;
    }
    c->n_vocab = n_vocab;
    return GEIST_HIP_OK;
}

/* The context of geist_sampler_argmax / _temperature lives under a thread-specific key whose
 * destructor gives the device memory back when the thread ends: a server that runs each
 * session on a short-lived thread (tests/test_multi_session_parallel_int.c:1-24) leaks
 * nothing. The main thread's context lives until the process ends. */
static pthread_key_t  g_ctx_key;
static pthread_once_t g_ctx_once = PTHREAD_ONCE_INIT;
static int            g_ctx_key_ok;

static void thread_ctx_destroy(void *p) {
    struct dropin_ctx *c = p;
    if (c != nullptr) {
        ctx_release(c);
        free(c);
    }
}

static void thread_ctx_key_make(void) {
    g_ctx_key_ok = pthread_key_create(&g_ctx_key, thread_ctx_destroy) == 0;
}

/* The calling thread's context for rows of n_vocab logits, or null after a reported failure. */
static struct dropin_ctx *thread_ctx(size_t n_vocab) {
    pthread_once(&g_ctx_once, thread_ctx_key_make);
    if (!g_ctx_key_ok) {
        fail("no thread-specific key for the device workspace", nullptr);
        return nullptr;
    }
    struct dropin_ctx *c = pthread_getspecific(g_ctx_key);
    if (c == nullptr) {
        c = calloc(1, sizeof *c);
        if (c == nullptr || pthread_setspecific(g_ctx_key, c) != 0) {
            free(c);
            fail("no memory for this thread's device workspace", nullptr);
            return nullptr;
        }
    }
    if (c->hs == nullptr || c->n_vocab < n_vocab) {
        ctx_release(c);
        if (ctx_setup(c, n_vocab) != GEIST_HIP_OK) {
            fail("no device workspace for this thread", nullptr);
            return nullptr;
        }
    }
    return c;
}

/* One row through the device path with the reference's precedence. */
static geist_token_t sample_one(struct dropin_ctx *c, size_t n, const float *logits,
                                float temperature, int top_k, float top_p, const float *u) {
    if (c == nullptr) /* the failure has been reported */
        return GEIST_SAMPLER_DROPIN_FAILED_TOKEN;
    if (geist_hip_upload(c->hs, c->d_row, logits, n * sizeof(float)) != GEIST_HIP_OK)
        return fail("upload of the logit row", c->hs);
    if (u != nullptr)
        *c->d_u = *u;
    const struct geist_hip_rows rows = {
        .d_logits = c->d_row, .ld = n, .rows = 1, .n_vocab = n};
    const struct geist_hip_sample_params prm = {.temperature        = temperature,
                                                .top_p              = top_p,
                                                .top_k              = top_k,
                                                .repetition_penalty = 1.0f,
                                                .precedence = GEIST_HIP_PRECEDENCE_REFERENCE};
    if (geist_hip_sample_rows(c->hs, &rows, &prm, u != nullptr ? c->d_u : nullptr, c->d_out) !=
        GEIST_HIP_OK)
        return fail("sampling", c->hs);
    if (geist_hip_sampler_sync(c->hs) != GEIST_HIP_OK)
        return fail("waiting for the token id", c->hs);
    return *c->d_out;
}

/* ---- RNG: sampler.c:27-48, exact integer arithmetic, stays on the host -------------------- */
void geist_rng_seed(struct geist_rng *rng, uint64_t seed) {
    if (rng == nullptr)
        return;
    rng->state = seed != 0 ? seed : UINT64_C(0x9E3779B97F4A7C15);
}

uint64_t geist_rng_next_u64(struct geist_rng *rng) {
    uint64_t s = rng->state;
    s ^= s >> 12;
    s ^= s << 25;
    s ^= s >> 27;
    rng->state = s;
    return s * UINT64_C(0x2545F4914F6CDD1D);
}

float geist_rng_next_unit(struct geist_rng *rng) {
    return (float) (uint32_t) (geist_rng_next_u64(rng) >> 40) * (1.0f / 16777216.0f);
}

/* ---- samplers ------------------------------------------------------------------------------ */
geist_token_t geist_sampler_argmax(size_t n_vocab, const float *logits) {
    return sample_one(thread_ctx(n_vocab), n_vocab, logits, 0.0f, 0, 1.0f, nullptr);
}

geist_token_t geist_sampler_temperature(size_t n_vocab, const float *logits, float temperature,
                                        struct geist_rng *rng) {
    struct dropin_ctx *c = thread_ctx(n_vocab);
    if (temperature <= 0.0f) /* sampler.c:110-112: greedy, no draw */
        return sample_one(c, n_vocab, logits, 0.0f, 0, 1.0f, nullptr);
    const float u = geist_rng_next_unit(rng); /* sampler.c:92: the one draw of this call */
    return sample_one(c, n_vocab, logits, temperature, 0, 1.0f, &u);
}

enum geist_status geist_sampler_workspace_init(struct geist_sampler_workspace *ws, size_t n_vocab) {
    if (ws == nullptr || n_vocab == 0)
        return GEIST_E_INVALID_ARG; /* sampler.c:138-140 */
    struct ws_header *h = aligned_alloc(64, (sizeof *h + n_vocab * sizeof(float) + 63) / 64 * 64);
    if (h == nullptr) {
        ws->probs   = nullptr;
        ws->n_vocab = 0;
        return GEIST_E_OOM; /* sampler.c:142-145 */
    }
    const int rc = ctx_setup(&h->ctx, n_vocab);
    if (rc != GEIST_HIP_OK) {
        free(h);
        ws->probs   = nullptr;
        ws->n_vocab = 0;
        return rc == GEIST_HIP_E_OOM ? GEIST_E_OOM : GEIST_E_BACKEND;
    }
    h->magic    = DROPIN_MAGIC;
    ws->probs   = (float *) (h + 1);
    ws->n_vocab = n_vocab;
    return GEIST_OK;
}

void geist_sampler_workspace_destroy(struct geist_sampler_workspace *ws) {
    if (ws == nullptr)
        return;
    if (ws->probs != nullptr) {
        struct ws_header *h = (struct ws_header *) ws->probs - 1;
        if (h->magic == DROPIN_MAGIC) {
            ctx_release(&h->ctx);
            h->magic = 0;
            free(h);
        }
        ws->probs = nullptr;
    }
    ws->n_vocab = 0; /* sampler.c:150-157: idempotent */
}

static struct dropin_ctx *ws_ctx(struct geist_sampler_workspace *ws) {
    struct ws_header *h = ws->probs != nullptr ? (struct ws_header *) ws->probs - 1 : nullptr;
    if (h == nullptr || h->magic != DROPIN_MAGIC) {
        fail("workspace was not made by geist_sampler_workspace_init", nullptr);
        return nullptr;
    }
    return &h->ctx;
}

geist_token_t geist_sampler_top_k_ws(struct geist_sampler_workspace *ws, const float *logits,
                                     int top_k, float temperature, struct geist_rng *rng) {
    struct dropin_ctx *c = ws_ctx(ws);
    const size_t       n = ws->n_vocab;
    if (top_k <= 1 || temperature <= 0.0f) /* sampler.c:184-186 */
        return sample_one(c, n, logits, 0.0f, 0, 1.0f, nullptr);
    /* sampler.c:187-189 sends top_k >= n to the temperature sampler; the device dispatch does
     * the same, and either way exactly one draw is taken */
    const float u = geist_rng_next_unit(rng);
    return sample_one(c, n, logits, temperature, top_k, 1.0f, &u);
}

geist_token_t geist_sampler_top_p_ws(struct geist_sampler_workspace *ws, const float *logits,
                                     float top_p, float temperature, struct geist_rng *rng) {
    struct dropin_ctx *c = ws_ctx(ws);
    const size_t       n = ws->n_vocab;
    if (top_p <= 0.0f || temperature <= 0.0f) /* sampler.c:238-240 */
        return sample_one(c, n, logits, 0.0f, 0, 1.0f, nullptr);
    const float u = geist_rng_next_unit(rng); /* sampler.c:242 or :290: one draw */
    return sample_one(c, n, logits, temperature, 0, top_p, &u);
}
