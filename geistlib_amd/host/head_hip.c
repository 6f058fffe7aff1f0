/*
 * head_hip.c -- sampler state of a session and the sampler dispatch of the output head, for
 * logits resident in device memory (C23). See include/geist_head_hip.h for the map onto the
 * reference's functions.
 */
#include "geist_head_hip.h"
#include "geist_sampler_hip.h"
#include "geist_lm_head_hip.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

struct geist_hip_head {
    /* src/archs/transformer/arch_state.h:287-294 */
    float    temperature;
    float    top_p;
    int      top_k;
    float    logit_softcap;
    size_t   vocab;
    size_t   m_max;
    geist_hip_sampler *hs;
    uint64_t *d_rng;   /* the session's struct geist_rng, in device memory */
    /* d_tokens, d_nacc, d_ngram and d_spec_result are page-locked host memory that the device
     * writes in place (geist_hip_host_malloc): reading them takes a wait for the stream and no
     * copy command (read_back) */
    int32_t  *d_tokens; /* m_max */
    float    *d_units;  /* m_max uniforms of one speculative round */
    int32_t  *d_drafts; /* m_max */
    int32_t  *d_nacc;
    int32_t  *d_ngram;  /* seed, history length, count, matched length, 16 drafts */
    void       *d_q6k_packed; /* the Q6_K table of geist_hip_head_q6k_load, repacked */
    const void *q6k_source;   /* ... the table it was packed from, and its row length */
    size_t      q6k_d_model;
    void       *d_q4k_packed; /* the same for a Q4_K table (geist_hip_head_q4k_load) */
    const void *q4k_source;
    size_t      q4k_d_model;
    float    *d_normed; /* m_max x d_model_cap: the normed hidden rows */
    size_t    d_model_cap;
    float    *d_logits; /* m_max x vocab, written by the lm_head, read by the sampler */
    bool      logits_sparse; /* the last token came from the sketch head: no dense logits */
    geist_hip_spec_head          *spec;        /* sketch of the tied table, or nullptr */
    struct geist_hip_spec_result *d_spec_result;
    size_t                        spec_d_model;
    char      err[256];
};

static int head_fail(struct geist_hip_head *h, int code, const char *what) {
    if (h != nullptr)
        snprintf(h->err, sizeof h->err, "%s: %s", what,
                 h->hs != nullptr ? geist_hip_sampler_last_error(h->hs) : "");
    return code;
}

/* What the kernels queued so far have left in one of the page-locked result buffers. */
static int read_back(struct geist_hip_head *h, void *dst, const void *pinned, size_t bytes) {
    if (geist_hip_sampler_sync(h->hs) != GEIST_HIP_OK)
        return GEIST_HIP_E_BACKEND;
    memcpy(dst, pinned, bytes);
    return GEIST_HIP_OK;
}

/* The token ids of the sampling call enqueued last: the call returns with the tokens, as the
 * reference's does (forward/head.c:165-186), as soon as the kernels have written them -- the
 * sampler reports that into page-locked memory (geist_hip_sampler_notify_ids), and only a call
 * that is not reported in time waits for the stream. */
static int read_ids(struct geist_hip_head *h, void *dst, const void *pinned, size_t bytes) {
    if (geist_hip_sampler_wait_ids(h->hs) != GEIST_HIP_OK)
        return GEIST_HIP_E_BACKEND;
    memcpy(dst, pinned, bytes);
    return GEIST_HIP_OK;
}

static int seed_rng(struct geist_hip_head *h, uint64_t seed) {
    /* geist_rng_seed, src/engine/sampler.c:27-33 */
    const uint64_t state = seed != 0 ? seed : UINT64_C(0x9E3779B97F4A7C15);
    return geist_hip_upload(h->hs, h->d_rng, &state, sizeof state);
}

int geist_hip_head_create(int device, size_t vocab, size_t m_max, float logit_softcap,
                          void *stream, struct geist_hip_head **out) {
    if (out == nullptr || vocab == 0)
        return GEIST_HIP_E_INVALID_ARG;
    *out                     = nullptr;
    struct geist_hip_head *h = calloc(1, sizeof *h);
    if (h == nullptr)
        return GEIST_HIP_E_OOM;
    h->vocab         = vocab;
    h->m_max         = m_max != 0 ? m_max : 64; /* include/geist.h:244-246 */
    h->logit_softcap = logit_softcap;
    /* sampler defaults: greedy (arch_state.c:1168-1171) */
    h->temperature = 0.0f;
    h->top_p       = 1.0f;
    h->top_k       = 0;
    int rc         = geist_hip_sampler_create(device, h->m_max, vocab, stream, &h->hs);
    void *p        = nullptr;
    if (rc == GEIST_HIP_OK && (rc = geist_hip_malloc(h->hs, sizeof(uint64_t), &p)) == GEIST_HIP_OK)
        h->d_rng = p;
    if (rc == GEIST_HIP_OK &&
        (rc = geist_hip_host_malloc(h->hs, h->m_max * sizeof(int32_t), &p)) == GEIST_HIP_OK)
        h->d_tokens = p;
    if (rc == GEIST_HIP_OK &&
        (rc = geist_hip_malloc(h->hs, h->m_max * sizeof(float), &p)) == GEIST_HIP_OK)
        h->d_units = p;
    if (rc == GEIST_HIP_OK &&
        (rc = geist_hip_malloc(h->hs, h->m_max * sizeof(int32_t), &p)) == GEIST_HIP_OK)
        h->d_drafts = p;
    if (rc == GEIST_HIP_OK &&
        (rc = geist_hip_host_malloc(h->hs, sizeof(int32_t), &p)) == GEIST_HIP_OK)
        h->d_nacc = p;
    if (rc == GEIST_HIP_OK &&
        (rc = geist_hip_host_malloc(h->hs, 20 * sizeof(int32_t), &p)) == GEIST_HIP_OK)
        h->d_ngram = p;
    if (rc == GEIST_HIP_OK)
        rc = geist_hip_sampler_notify_ids(h->hs, 1); /* see read_ids() */
    /* arch_state.c:1173: the default seed */
    if (rc == GEIST_HIP_OK)
        rc = seed_rng(h, UINT64_C(0xCAFEBABE1234));
    if (rc != GEIST_HIP_OK) {
        geist_hip_head_destroy(h);
        return rc;
    }
    *out = h;
    return GEIST_HIP_OK;
}

void geist_hip_head_destroy(struct geist_hip_head *h) {
    if (h == nullptr)
        return;
    if (h->hs != nullptr) {
        geist_hip_free(h->hs, h->d_rng);
        geist_hip_host_free(h->hs, h->d_tokens);
        geist_hip_free(h->hs, h->d_units);
        geist_hip_free(h->hs, h->d_drafts);
        geist_hip_host_free(h->hs, h->d_nacc);
        geist_hip_host_free(h->hs, h->d_ngram);
        geist_hip_free(h->hs, h->d_normed);
        geist_hip_free(h->hs, h->d_q6k_packed);
        geist_hip_free(h->hs, h->d_q4k_packed);
        geist_hip_free(h->hs, h->d_logits);
        geist_hip_host_free(h->hs, h->d_spec_result);
        geist_hip_spec_head_destroy(h->hs, h->spec);
        geist_hip_sampler_destroy(h->hs);
    }
    free(h);
}

const char *geist_hip_head_errmsg(const struct geist_hip_head *h) { return h ? h->err : ""; }

/* The session's sampling options as the device layer takes them: the reference's precedence,
 * no penalties, the model's soft-cap. */
static struct geist_hip_sample_params head_params(const struct geist_hip_head *h) {
    return (struct geist_hip_sample_params) {.temperature        = h->temperature,
                                             .top_p              = h->top_p,
                                             .top_k              = h->top_k,
                                             .repetition_penalty = 1.0f,
                                             .logit_softcap      = h->logit_softcap,
                                             .precedence = GEIST_HIP_PRECEDENCE_REFERENCE};
}

int geist_hip_head_apply_opts(struct geist_hip_head *h, const struct geist_session_opts *opts) {
    if (h == nullptr)
        return GEIST_HIP_E_INVALID_ARG;
    if (opts == nullptr)
        return GEIST_HIP_OK; /* geist_session_create with NULL opts: greedy defaults stay */
    /* step.c:390-396 */
    h->temperature = opts->temperature;
    h->top_p       = opts->top_p > 0.0f ? opts->top_p : 1.0f;
    h->top_k       = opts->top_k;
    if (opts->random_seed != 0 && seed_rng(h, opts->random_seed) != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_BACKEND, "seeding the device RNG");
    /* step.c:398-409 sizes the sampler workspace here, once top_p is known, so that no decode
     * step allocates; so does this */
    const struct geist_hip_sample_params prm = head_params(h);
    if (geist_hip_sampler_prepare(h->hs, &prm, h->vocab) != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_OOM, "sampler workspace");
    return GEIST_HIP_OK;
}

/* The [m_max, vocab] logit buffer and the normed rows; *grown says whether d_model outgrew what
 * was there. */
static int reserve_head_buffers(struct geist_hip_head *h, size_t d_model, bool *grown) {
    *grown = false;
    if (h == nullptr || d_model == 0)
        return GEIST_HIP_E_INVALID_ARG;
    void *p = nullptr;
    if (h->d_logits == nullptr) {
        if (geist_hip_malloc(h->hs, h->m_max * h->vocab * sizeof(float), &p) != GEIST_HIP_OK)
            return head_fail(h, GEIST_HIP_E_OOM, "logit buffer");
        h->d_logits = p;
    }
    if (h->d_model_cap < d_model) {
        geist_hip_free(h->hs, h->d_normed);
        h->d_normed    = nullptr;
        h->d_model_cap = 0;
        if (geist_hip_malloc(h->hs, h->m_max * d_model * sizeof(float), &p) != GEIST_HIP_OK)
            return head_fail(h, GEIST_HIP_E_OOM, "buffer of normed rows");
        h->d_normed    = p;
        h->d_model_cap = d_model;
        *grown         = true;
    }
    return GEIST_HIP_OK;
}

int geist_hip_head_reserve_projection(struct geist_hip_head *h, size_t d_model) {
    bool      grown;
    const int rc = reserve_head_buffers(h, d_model, &grown);
    if (rc != GEIST_HIP_OK)
        return rc;
    /* a batch of rows goes through the double-precision projection, which has scratch */
    if (grown && h->m_max > 1 && d_model % 8 == 0 &&
        geist_hip_f16_linear_reserve(h->hs, h->vocab, d_model) != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_OOM, "scratch of the batch projection");
    return GEIST_HIP_OK;
}

static int finalize(struct geist_hip_head *h, const float *d_logits, size_t k, int32_t *out) {
    if (h == nullptr || d_logits == nullptr || out == nullptr || k == 0)
        return GEIST_HIP_E_INVALID_ARG;
    if (k > h->m_max)
        return head_fail(h, GEIST_HIP_E_INVALID_ARG, "more rows than m_max");
    const struct geist_hip_rows rows = {
        .d_logits = d_logits, .ld = h->vocab, .rows = k, .n_vocab = h->vocab};
    /* head.c:172-183 / 291-302: T == 0 -> argmax; top_k > 1 -> top-k; 0 < top_p < 1 -> top-p;
     * else temperature. Rows in order, one shared RNG (head.c:274-304). */
    const struct geist_hip_sample_params prm = head_params(h);
    if (geist_hip_sample_rows_rng(h->hs, &rows, &prm, h->d_rng, /*shared=*/1, h->d_tokens) !=
        GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_BACKEND, "sampling");
    if (read_ids(h, out, h->d_tokens, k * sizeof(int32_t)) != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_BACKEND, "reading back the token ids");
    for (size_t r = 0; r < k; r++) /* head.c:137-139: an id outside the vocabulary is an error */
        if (out[r] < 0 || (size_t) out[r] >= h->vocab)
            return head_fail(h, GEIST_HIP_E_BACKEND, "token id out of range");
    return GEIST_HIP_OK;
}

int geist_hip_head_finalize_one_row(struct geist_hip_head *h, const float *d_logits,
                                    int32_t *out_token) {
    return finalize(h, d_logits, 1, out_token);
}

int geist_hip_head_finalize_batch(struct geist_hip_head *h, const float *d_logits, size_t k,
                                  int32_t *out_tokens) {
    return finalize(h, d_logits, k, out_tokens);
}

static int project_finalize_table(struct geist_hip_head *h, const float *d_hidden,
                                  size_t ld_hidden, size_t k, const float *d_norm_weight,
                                  float rms_eps, const void *d_embed, const float *d_scales,
                                  bool q6k, size_t d_model, int32_t *out_tokens);

/* The table is binary16 (d_scales == nullptr), int8 with one scale per row, or Q6_K blocks. */
static int project_finalize(struct geist_hip_head *h, const float *d_hidden, size_t ld_hidden,
                            size_t k, const float *d_norm_weight, float rms_eps,
                            const void *d_embed, const float *d_scales, size_t d_model,
                            int32_t *out_tokens) {
    return project_finalize_table(h, d_hidden, ld_hidden, k, d_norm_weight, rms_eps, d_embed,
                                  d_scales, false, d_model, out_tokens);
}

static int project_finalize_table(struct geist_hip_head *h, const float *d_hidden,
                                  size_t ld_hidden, size_t k, const float *d_norm_weight,
                                  float rms_eps, const void *d_embed, const float *d_scales,
                                  bool q6k, size_t d_model, int32_t *out_tokens) {
    if (h == nullptr || d_hidden == nullptr || d_norm_weight == nullptr || d_embed == nullptr ||
        out_tokens == nullptr || k == 0 || d_model == 0)
        return GEIST_HIP_E_INVALID_ARG;
    if (k > h->m_max)
        return head_fail(h, GEIST_HIP_E_INVALID_ARG, "more rows than m_max");
    /* a no-op after geist_hip_head_reserve_projection[_q6k] with this d_model */
    const int rrc = q6k ? geist_hip_head_reserve_projection_q6k(h, d_model)
                        : geist_hip_head_reserve_projection(h, d_model);
    if (rrc != GEIST_HIP_OK)
        return rrc;
    /* head.c:99-101, 114-126, then the dispatch of 172-183 / 291-302 with the session's RNG */
    const struct geist_hip_sample_params prm = head_params(h);
    /* the table that geist_hip_head_q6k_load repacked is read from its packed copy */
    const bool packed = q6k && h->d_q6k_packed != nullptr && d_embed == h->q6k_source &&
                        d_model == h->q6k_d_model;
    const int rc =
            packed ? geist_hip_project_sample_rows_q6k_packed(
                             h->hs, d_hidden, ld_hidden, k, d_model, d_norm_weight, rms_eps,
                             h->d_q6k_packed, h->vocab, h->d_normed, h->d_logits, h->vocab, &prm,
                             nullptr, h->d_rng, /*shared=*/1, h->d_tokens)
            : q6k ? geist_hip_project_sample_rows_q6k(h->hs, d_hidden, ld_hidden, k, d_model,
                                                      d_norm_weight, rms_eps, d_embed, h->vocab,
                                                      h->d_normed, h->d_logits, h->vocab, &prm,
                                                      nullptr, h->d_rng, /*shared=*/1, h->d_tokens)
            : d_scales != nullptr
                    ? geist_hip_project_sample_rows_q8w(h->hs, d_hidden, ld_hidden, k, d_model,
                                                        d_norm_weight, rms_eps, d_embed, d_scales,
                                                        h->vocab, h->d_normed, h->d_logits,
                                                        h->vocab, &prm, nullptr, h->d_rng,
                                                        /*shared=*/1, h->d_tokens)
                    : geist_hip_project_sample_rows(h->hs, d_hidden, ld_hidden, k, d_model,
                                                    d_norm_weight, rms_eps, d_embed, h->vocab,
                                                    h->d_normed, h->d_logits, h->vocab, &prm,
                                                    nullptr, h->d_rng, /*shared=*/1, h->d_tokens);
    if (rc != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_BACKEND, "output head");
    h->logits_sparse = false;
    if (read_ids(h, out_tokens, h->d_tokens, k * sizeof(int32_t)) != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_BACKEND, "reading back the token ids");
    for (size_t r = 0; r < k; r++)
        if (out_tokens[r] < 0 || (size_t) out_tokens[r] >= h->vocab)
            return head_fail(h, GEIST_HIP_E_BACKEND, "token id out of range");
    return GEIST_HIP_OK;
}

int geist_hip_head_project_finalize_q6k(struct geist_hip_head *h, const float *d_hidden,
                                        size_t ld_hidden, size_t k, const float *d_norm_weight,
                                        float rms_eps, const void *d_embed_q6k, size_t d_model,
                                        int32_t *out_tokens) {
    return project_finalize_table(h, d_hidden, ld_hidden, k, d_norm_weight, rms_eps, d_embed_q6k,
                                  nullptr, true, d_model, out_tokens);
}

int geist_hip_head_q6k_load(struct geist_hip_head *h, const void *d_embed_q6k, size_t d_model) {
    if (h == nullptr || d_embed_q6k == nullptr || d_model == 0)
        return GEIST_HIP_E_INVALID_ARG;
    const size_t bytes = geist_hip_q6k_packed_bytes(h->vocab, d_model);
    if (bytes == 0)
        return head_fail(h, GEIST_HIP_E_UNSUPPORTED, "Q6_K table: d_model not a multiple of 256");
    geist_hip_free(h->hs, h->d_q6k_packed);
    h->d_q6k_packed = nullptr;
    h->q6k_source   = nullptr;
    void *p         = nullptr;
    if (geist_hip_malloc(h->hs, bytes, &p) != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_OOM, "packed Q6_K table");
    if (geist_hip_q6k_pack(h->hs, d_embed_q6k, h->vocab, d_model, p) != GEIST_HIP_OK ||
        geist_hip_sampler_sync(h->hs) != GEIST_HIP_OK) {
        geist_hip_free(h->hs, p);
        return head_fail(h, GEIST_HIP_E_BACKEND, "packing the Q6_K table");
    }
    h->d_q6k_packed = p;
    h->q6k_source   = d_embed_q6k;
    h->q6k_d_model  = d_model;
    return geist_hip_head_reserve_projection_q6k(h, d_model);
}

/* Q4_K: only the packed copy has a kernel, so the table has to have been loaded. */
int geist_hip_head_project_finalize_q4k(struct geist_hip_head *h, const float *d_hidden,
                                        size_t ld_hidden, size_t k, const float *d_norm_weight,
                                        float rms_eps, const void *d_embed_q4k, size_t d_model,
                                        int32_t *out_tokens) {
    if (h == nullptr || d_hidden == nullptr || d_norm_weight == nullptr || d_embed_q4k == nullptr ||
        out_tokens == nullptr || k == 0 || d_model == 0)
        return GEIST_HIP_E_INVALID_ARG;
    if (k > h->m_max)
        return head_fail(h, GEIST_HIP_E_INVALID_ARG, "more rows than m_max");
    if (h->d_q4k_packed == nullptr || d_embed_q4k != h->q4k_source || d_model != h->q4k_d_model)
        return head_fail(h, GEIST_HIP_E_UNSUPPORTED,
                         "Q4_K table not loaded (geist_hip_head_q4k_load)");
    const int rrc = geist_hip_head_reserve_projection_q6k(h, d_model); /* a no-op after the load */
    if (rrc != GEIST_HIP_OK)
        return rrc;
    const struct geist_hip_sample_params prm = head_params(h);
    const int rc = geist_hip_project_sample_rows_q4k_packed(
            h->hs, d_hidden, ld_hidden, k, d_model, d_norm_weight, rms_eps, h->d_q4k_packed,
            h->vocab, h->d_normed, h->d_logits, h->vocab, &prm, nullptr, h->d_rng, /*shared=*/1,
            h->d_tokens);
    if (rc != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_BACKEND, "output head");
    h->logits_sparse = false;
    if (read_ids(h, out_tokens, h->d_tokens, k * sizeof(int32_t)) != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_BACKEND, "reading back the token ids");
    for (size_t r = 0; r < k; r++)
        if (out_tokens[r] < 0 || (size_t) out_tokens[r] >= h->vocab)
            return head_fail(h, GEIST_HIP_E_BACKEND, "token id out of range");
    return GEIST_HIP_OK;
}

int geist_hip_head_q4k_load(struct geist_hip_head *h, const void *d_embed_q4k, size_t d_model) {
    if (h == nullptr || d_embed_q4k == nullptr || d_model == 0)
        return GEIST_HIP_E_INVALID_ARG;
    const size_t bytes = geist_hip_q4k_packed_bytes(h->vocab, d_model);
    if (bytes == 0)
        return head_fail(h, GEIST_HIP_E_UNSUPPORTED, "Q4_K table: d_model not a multiple of 256");
    geist_hip_free(h->hs, h->d_q4k_packed);
    h->d_q4k_packed = nullptr;
    h->q4k_source   = nullptr;
    void *p         = nullptr;
    if (geist_hip_malloc(h->hs, bytes, &p) != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_OOM, "packed Q4_K table");
    if (geist_hip_q4k_pack(h->hs, d_embed_q4k, h->vocab, d_model, p) != GEIST_HIP_OK ||
        geist_hip_sampler_sync(h->hs) != GEIST_HIP_OK) {
        geist_hip_free(h->hs, p);
        return head_fail(h, GEIST_HIP_E_BACKEND, "packing the Q4_K table");
    }
    h->d_q4k_packed = p;
    h->q4k_source   = d_embed_q4k;
    h->q4k_d_model  = d_model;
    return geist_hip_head_reserve_projection_q6k(h, d_model); /* the same buffers and scratch */
}

int geist_hip_head_reserve_projection_q6k(struct geist_hip_head *h, size_t d_model) {
    bool      grown;
    const int rc = reserve_head_buffers(h, d_model, &grown);
    if (rc != GEIST_HIP_OK)
        return rc;
    if (geist_hip_q6k_linear_reserve(h->hs, h->vocab, d_model) != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_OOM, "scratch of the Q6_K projection");
    return GEIST_HIP_OK;
}

int geist_hip_head_set_sums(struct geist_hip_head *h, int mode) {
    if (h == nullptr)
        return GEIST_HIP_E_INVALID_ARG;
    if (geist_hip_sampler_set_sums(h->hs, mode) != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_INVALID_ARG, "sums mode");
    return GEIST_HIP_OK;
}

int geist_hip_head_set_projection(struct geist_hip_head *h, int mode) {
    if (h == nullptr)
        return GEIST_HIP_E_INVALID_ARG;
    if (geist_hip_sampler_set_projection(h->hs, mode) != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_INVALID_ARG, "projection mode");
    return GEIST_HIP_OK;
}

int geist_hip_head_project_finalize(struct geist_hip_head *h, const float *d_hidden,
                                    size_t ld_hidden, size_t k, const float *d_norm_weight,
                                    float rms_eps, const uint16_t *d_embed_f16, size_t d_model,
                                    int32_t *out_tokens) {
    return project_finalize(h, d_hidden, ld_hidden, k, d_norm_weight, rms_eps, d_embed_f16, nullptr,
                            d_model, out_tokens);
}

int geist_hip_head_project_finalize_q8w(struct geist_hip_head *h, const float *d_hidden,
                                        size_t ld_hidden, size_t k, const float *d_norm_weight,
                                        float rms_eps, const int8_t *d_embed_q8,
                                        const float *d_scales, size_t d_model,
                                        int32_t *out_tokens) {
    if (d_scales == nullptr)
        return GEIST_HIP_E_INVALID_ARG;
    return project_finalize(h, d_hidden, ld_hidden, k, d_norm_weight, rms_eps, d_embed_q8, d_scales,
                            d_model, out_tokens);
}

int geist_hip_head_spec_build(struct geist_hip_head *h, const uint16_t *d_embed_f16, size_t d_model,
                              size_t stride_override, size_t topk_override) {
    if (h == nullptr || d_embed_f16 == nullptr || d_model == 0)
        return GEIST_HIP_E_INVALID_ARG;
    geist_hip_spec_head_destroy(h->hs, h->spec);
    h->spec = nullptr;
    void *p = nullptr;
    if (h->d_spec_result == nullptr) {
        if (geist_hip_host_malloc(h->hs, sizeof *h->d_spec_result, &p) != GEIST_HIP_OK)
            return head_fail(h, GEIST_HIP_E_OOM, "sketch head result");
        h->d_spec_result = p;
    }
    /* transformer_spec_head_init, spec_head.c:616-622: a head that is not eligible simply has no
     * sketch; the caller keeps the dense path */
    const int rc = geist_hip_spec_head_build(h->hs, d_embed_f16, h->vocab, d_model, stride_override,
                                             topk_override, &h->spec);
    if (rc != GEIST_HIP_OK)
        return head_fail(h, rc, "sketch head");
    h->spec_d_model = d_model;
    return GEIST_HIP_OK;
}

int geist_hip_head_project_finalize_spec(struct geist_hip_head *h, const float *d_hidden,
                                         const float *d_norm_weight, float rms_eps,
                                         const uint16_t *d_embed_f16, size_t d_model, int verify,
                                         int32_t *out_token, int *used_sketch) {
    if (h == nullptr || d_hidden == nullptr || d_norm_weight == nullptr || d_embed_f16 == nullptr ||
        out_token == nullptr || d_model == 0)
        return GEIST_HIP_E_INVALID_ARG;
    if (used_sketch != nullptr)
        *used_sketch = 0;
    /* spec_head.c:645-647: greedy only; spec_state != 1: no sketch */
    if (h->spec == nullptr || h->temperature != 0.0f || d_model != h->spec_d_model)
        return project_finalize(h, d_hidden, d_model, 1, d_norm_weight, rms_eps, d_embed_f16,
                                nullptr, d_model, out_token);
    if (h->d_model_cap < d_model) {
        const int rrc = geist_hip_head_reserve_projection(h, d_model);
        if (rrc != GEIST_HIP_OK)
            return rrc;
    }
    /* head.c:99-101, then head.c:109 */
    struct geist_hip_spec_result res;
    if (geist_hip_spec_head_try_hidden(h->hs, h->spec, d_hidden, d_norm_weight, rms_eps,
                                       h->d_normed, verify, h->d_spec_result) != GEIST_HIP_OK ||
        read_back(h, &res, h->d_spec_result, sizeof res) != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_BACKEND, "sketch head");
    if (res.answered == 0) /* head.c:114-188: the dense head */
        return project_finalize(h, d_hidden, d_model, 1, d_norm_weight, rms_eps, d_embed_f16,
                                nullptr, d_model, out_token);
    if (res.token < 0 || (size_t) res.token >= h->vocab)
        return head_fail(h, GEIST_HIP_E_BACKEND, "token id out of range");
    *out_token       = res.token;
    h->logits_sparse = true; /* spec_head.c:880 */
    if (used_sketch != nullptr)
        *used_sketch = 1;
    return GEIST_HIP_OK;
}

const float *geist_hip_head_logits(const struct geist_hip_head *h) {
    return h != nullptr && !h->logits_sparse ? h->d_logits : nullptr;
}

int geist_hip_head_argmax_f32(struct geist_hip_head *h, const float *d_logits, size_t n,
                              int32_t *out_index) {
    if (h == nullptr)
        return GEIST_HIP_E_INVALID_ARG;
    if (n > h->vocab) /* geist_backend.h:322-326: outside the probed geometry */
        return head_fail(h, GEIST_HIP_E_UNSUPPORTED, "row longer than the probed vocabulary");
    if (geist_hip_argmax_f32(h->hs, d_logits, n, out_index) != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_BACKEND, "argmax");
    return GEIST_HIP_OK;
}

int geist_hip_head_propose_drafts(struct geist_hip_head *h, const int32_t *d_history,
                                  size_t history_n, int32_t seed, size_t k_max,
                                  int32_t *out_drafts, size_t *n_drafts, size_t *match_len) {
    if (h == nullptr || out_drafts == nullptr || n_drafts == nullptr ||
        (history_n > 0 && d_history == nullptr))
        return GEIST_HIP_E_INVALID_ARG;
    *n_drafts = 0;
    if (match_len != nullptr)
        *match_len = 0;
    if (k_max == 0 || k_max > 16) /* session.c:546-548 */
        return head_fail(h, GEIST_HIP_E_INVALID_ARG, "k_max outside 1..16");
    if (history_n > INT32_MAX)
        return head_fail(h, GEIST_HIP_E_INVALID_ARG, "history too long");
    out_drafts[0] = seed;
    *n_drafts     = 1;
    if (history_n == 0 || k_max == 1) /* session.c:446-447 */
        return GEIST_HIP_OK;
    int32_t back[18];
    h->d_ngram[0] = seed; /* the kernel reads both in place */
    h->d_ngram[1] = (int32_t) history_n;
    if (geist_hip_propose_drafts_ngram(h->hs, d_history, history_n, h->d_ngram + 1, h->d_ngram, 1,
                                       k_max, /*max_suffix=*/4, h->d_ngram + 4, 16,
                                       h->d_ngram + 2, h->d_ngram + 3) != GEIST_HIP_OK ||
        read_back(h, back, h->d_ngram + 2, (2 + k_max) * sizeof(int32_t)) != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_BACKEND, "n-gram drafts");
    if (back[0] < 1 || (size_t) back[0] > k_max || back[1] < 0 || back[1] > 4)
        return head_fail(h, GEIST_HIP_E_BACKEND, "draft count out of range");
    memcpy(out_drafts, back + 2, (size_t) back[0] * sizeof *out_drafts);
    *n_drafts = (size_t) back[0];
    if (match_len != nullptr)
        *match_len = (size_t) back[1];
    return GEIST_HIP_OK;
}

int geist_hip_head_spec_accept(struct geist_hip_head *h, const float *d_logits, size_t k,
                               const int32_t *drafts, int mode, size_t out_capacity,
                               int32_t *out_tokens, size_t *n_out) {
    if (h == nullptr || d_logits == nullptr || drafts == nullptr || out_tokens == nullptr ||
        n_out == nullptr || k == 0)
        return GEIST_HIP_E_INVALID_ARG;
    *n_out = 0;
    if (k > h->m_max)
        return head_fail(h, GEIST_HIP_E_INVALID_ARG, "more rows than m_max");
    if (out_capacity < k + 1)
        return head_fail(h, GEIST_HIP_E_INVALID_ARG, "out_capacity below k + 1");
    const bool greedy   = !(h->temperature > 0.0f);
    const bool filtered = h->top_k > 1 || (h->top_p > 0.0f && h->top_p < 1.0f);
    if (mode == GEIST_HIP_SPEC_REJECTION && !greedy && filtered)
        return head_fail(h, GEIST_HIP_E_UNSUPPORTED,
                         "rejection sampling against a top-k / top-p filtered target");
    if (mode != GEIST_HIP_SPEC_REJECTION || greedy || k == 1) {
        /* session.c:599-625: sample every row, accept the longest matching prefix */
        int32_t   sampled[64];
        int32_t  *v  = k <= 64 ? sampled : malloc(k * sizeof *v);
        if (v == nullptr)
            return GEIST_HIP_E_OOM;
        const int rc = finalize(h, d_logits, k, v);
        if (rc == GEIST_HIP_OK) {
            size_t accepted = 0;
            for (size_t i = 0; i + 1 < k; i++) {
                if (v[i] != drafts[i + 1])
                    break;
                accepted++;
            }
            memcpy(out_tokens, drafts, (accepted + 1) * sizeof *out_tokens);
            out_tokens[accepted + 1] = v[accepted];
            *n_out                   = accepted + 2;
        }
        if (v != sampled)
            free(v);
        return rc;
    }
    /* rejection sampling: L = k - 1 drafts (drafts[1..k)) against rows 0..L-1, bonus from row L */
    const size_t L = k - 1;
    if (geist_hip_upload(h->hs, h->d_drafts, drafts + 1, L * sizeof(int32_t)) != GEIST_HIP_OK ||
        geist_hip_rng_draw_units(h->hs, h->d_rng, k, h->d_units) != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_BACKEND, "staging the drafts");
    if (geist_hip_spec_verify(h->hs, d_logits, h->vocab, nullptr, 0, h->d_drafts, h->d_units, 1, L,
                              h->vocab, h->temperature, h->logit_softcap, h->d_tokens,
                              h->d_nacc) != GEIST_HIP_OK)
        return head_fail(h, GEIST_HIP_E_BACKEND, "verification");
    int32_t n_acc = 0;
    if (read_back(h, &n_acc, h->d_nacc, sizeof n_acc) != GEIST_HIP_OK || n_acc < 0 ||
        (size_t) n_acc > L)
        return head_fail(h, GEIST_HIP_E_BACKEND, "reading back the verdict");
    memcpy(out_tokens + 1, h->d_tokens, ((size_t) n_acc + 1) * sizeof(int32_t));
    out_tokens[0] = drafts[0];
    *n_out        = (size_t) n_acc + 2;
    for (size_t i = 0; i < *n_out; i++)
        if (out_tokens[i] < 0 || (size_t) out_tokens[i] >= h->vocab)
            return head_fail(h, GEIST_HIP_E_BACKEND, "token id out of range");
    return GEIST_HIP_OK;
}

int geist_hip_head_rng_state(struct geist_hip_head *h, uint64_t *state) {
    if (h == nullptr || state == nullptr)
        return GEIST_HIP_E_INVALID_ARG;
    return geist_hip_download(h->hs, state, h->d_rng, sizeof *state);
}
