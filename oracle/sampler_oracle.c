/*
 * sampler_oracle.c -- CPU restatement of the reference token sampler (see the header).
 *
 * TEST INFRASTRUCTURE ONLY: never linked into, loaded by or called from the shipped
 * library. Build: `make -C oracle` (strict IEEE, no contraction) and a second object with
 * the reference's release flags for the CPU timing leg.
 *
 * Pinned by tests/test_oracle_*.py against: the compiled reference (oracle/_ref, where
 * the reference tree is mounted), the committed golden vectors made from it, the eight
 * known-answer checks of the reference's tests/test_sampler_unit.c, and closed forms /
 * brute force for the stages the reference lacks.
 */
#include "sampler_oracle.h"

#include <math.h>
#include <stdbool.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ======================================================================================
 * RNG (src/engine/sampler.c:27-48): xorshift64* with the (12, 25, 27) triple.
 * ==================================================================================== */
void oracle_rng_seed(struct oracle_rng *rng, uint64_t seed) {
    if (!rng)
        return;
    rng->state = seed ? seed : UINT64_C(0x9E3779B97F4A7C15); /* sampler.c:32 */
}

uint64_t oracle_rng_next_u64(struct oracle_rng *rng) {
    uint64_t s = rng->state;
    s ^= s >> 12;
    s ^= s << 25;
    s ^= s >> 27;
    rng->state = s;
    return s * UINT64_C(0x2545F4914F6CDD1D);
}

float oracle_rng_next_unit(struct oracle_rng *rng) {
    /* sampler.c:44-48: the top 24 bits, scaled by 2^-24; exact in fp32. */
    uint32_t hi24 = (uint32_t) (oracle_rng_next_u64(rng) >> 40);
    return (float) hi24 * (1.0f / 16777216.0f);
}

/* A draw is either a fixed uniform or the next value of a caller-owned RNG; either way the
 * walk code below asks for it at the point where the reference calls geist_rng_next_unit. */
struct draw_src {
    struct oracle_rng *rng;
    float              u;
    int                taken;
};
static float take_draw(struct draw_src *d) {
    d->taken++;
    return d->rng ? oracle_rng_next_unit(d->rng) : d->u;
}

static void info_none(struct oracle_draw_info *info) {
    if (info) {
        info->boundary_dist = INFINITY;
        info->mass          = 0.0;
        info->n_keep        = 0;
        info->draws         = 0;
    }
}

/* ======================================================================================
 * argmax (sampler.c:52-62): first maximum wins, strict '>' so NaN can only win at index 0.
 * ==================================================================================== */
int32_t oracle_argmax(size_t n, const float *logits) {
    size_t at = 0;
    float  hi = logits[0];
    for (size_t i = 1; i < n; i++) {
        if (logits[i] > hi) {
            hi = logits[i];
            at = i;
        }
    }
    return (int32_t) at;
}

/* ======================================================================================
 * softmax_into (sampler.c:68-85): fp32 max, fp32 scaled difference, libm expf, and a double
 * sum accumulated in array order. Output stays un-normalised.
 * ==================================================================================== */
double oracle_softmax_into(size_t n, const float *logits, float temperature, float *probs) {
    float top = logits[0];
    for (size_t i = 1; i < n; i++)
        if (logits[i] > top)
            top = logits[i];
    const float inv_t = temperature > 0.0f ? 1.0f / temperature : 1.0f;
    double      total = 0.0;
    for (size_t i = 0; i < n; i++) {
        const float e = expf((logits[i] - top) * inv_t);
        probs[i]      = e;
        total += (double) e;
    }
    return total;
}

/* inv_cdf_sample (sampler.c:90-102) with the distance to the nearer slot edge recorded. */
static size_t walk_cdf(size_t n, const float *w, double mass, struct draw_src *d,
                       struct oracle_draw_info *info) {
    const double target = (double) take_draw(d) * mass;
    double       run    = 0.0;
    size_t       pick   = n - 1; /* rounding overflow: last entry (sampler.c:100-101) */
    double       lo = 0.0, hi = mass;
    int          found = 0;
    for (size_t i = 0; i < n; i++) {
        const double before = run;
        run += (double) w[i];
        if (target < run) {
            pick  = i;
            lo    = before;
            hi    = run;
            found = 1;
            break;
        }
    }
    if (info) {
        double dist = found ? fmin(target - lo, hi - target) : 0.0;
        info->boundary_dist = mass > 0.0 ? dist / mass : 0.0;
        info->mass          = mass;
        info->n_keep        = n;
        info->draws         = d->taken;
    }
    return pick;
}

/* ======================================================================================
 * temperature (sampler.c:106-132). The reference's stack-vs-heap split for the scratch
 * array has no arithmetic effect; one heap array serves both.
 * ==================================================================================== */
static int32_t temperature_core(size_t n, const float *logits, float temperature,
                                struct draw_src *d, struct oracle_draw_info *info) {
    if (temperature <= 0.0f) {
        info_none(info);
        return oracle_argmax(n, logits);
    }
    float *probs = (float *) malloc(n * sizeof(float));
    if (!probs) {
        info_none(info);
        return oracle_argmax(n, logits); /* sampler.c:125-127: no draw on this path */
    }
    const double sum  = oracle_softmax_into(n, logits, temperature, probs);
    const size_t pick = walk_cdf(n, probs, sum, d, info);
    free(probs);
    return (int32_t) pick;
}

/* ======================================================================================
 * Ordering used by top-k and top-p (sampler.c:162-176, 207, 270): key descending. Equal keys
 * keep ascending index (glibc 2.35 merge sort); NaN keys go last.
 * ==================================================================================== */
struct keyed {
    float    key;
    uint32_t idx;
};

/* 1 if a must come strictly before b. */
static int goes_first(const struct keyed *a, const struct keyed *b) {
    const int an = isnan(a->key), bn = isnan(b->key);
    if (an || bn) {
        if (an != bn)
            return bn; /* the number precedes the NaN */
        return a->idx < b->idx;
    }
    if (a->key > b->key)
        return 1;
    if (a->key < b->key)
        return 0;
    return a->idx < b->idx;
}

/* Bottom-up merge sort; stable by construction (and the index tiebreak makes it total). */
static int sort_desc(struct keyed *v, size_t n) {
    if (n < 2)
        return 0;
    struct keyed *tmp = (struct keyed *) malloc(n * sizeof *tmp);
    if (!tmp)
        return -1;
    struct keyed *src = v, *dst = tmp;
    for (size_t w = 1; w < n; w *= 2) {
        for (size_t lo = 0; lo < n; lo += 2 * w) {
            size_t mid = lo + w < n ? lo + w : n;
            size_t hi  = lo + 2 * w < n ? lo + 2 * w : n;
            size_t a = lo, b = mid, o = lo;
            while (a < mid && b < hi)
                dst[o++] = goes_first(&src[b], &src[a]) ? src[b++] : src[a++];
            while (a < mid)
                dst[o++] = src[a++];
            while (b < hi)
                dst[o++] = src[b++];
        }
        struct keyed *t = src;
        src             = dst;
        dst             = t;
    }
    if (src != v)
        memcpy(v, src, n * sizeof *v);
    free(tmp);
    return 0;
}

static struct keyed *keyed_from(size_t n, const float *vals) {
    struct keyed *v = (struct keyed *) malloc((n ? n : 1) * sizeof *v);
    if (!v)
        return NULL;
    for (size_t i = 0; i < n; i++) {
        v[i].key = vals[i];
        v[i].idx = (uint32_t) i;
    }
    return v;
}

#define ORACLE_TOPK_CAP 8192 /* sampler.c:210-215: stack budget of the reference */

/* ======================================================================================
 * top-k (sampler.c:178-228)
 * ==================================================================================== */
static int32_t top_k_core(size_t n, const float *logits, int top_k, float temperature,
                          struct draw_src *d, struct oracle_draw_info *info) {
    if (top_k <= 1 || temperature <= 0.0f) {
        info_none(info);
        return oracle_argmax(n, logits);
    }
    if ((size_t) top_k >= n)
        return temperature_core(n, logits, temperature, d, info);

    struct keyed *v = keyed_from(n, logits);
    if (!v || sort_desc(v, n) != 0) {
        free(v);
        info_none(info);
        return oracle_argmax(n, logits);
    }
    size_t k = (size_t) top_k;
    if (k > ORACLE_TOPK_CAP)
        k = ORACLE_TOPK_CAP;
    float *kl = (float *) malloc(2 * k * sizeof(float));
    float *kp = kl + k;
    for (size_t j = 0; j < k; j++)
        kl[j] = v[j].key;
    const double  sum  = oracle_softmax_into(k, kl, temperature, kp);
    const size_t  at   = walk_cdf(k, kp, sum, d, info);
    const int32_t pick = (int32_t) v[at].idx;
    free(kl);
    free(v);
    return pick;
}

/* ======================================================================================
 * Prefix selection + draw over an ordered weight list. Shared by top-p (sampler.c:272-299)
 * and by the chain. `w` are the (normalised) weights in walk order.
 *   top_p  in (0,1): nucleus = shortest prefix with running double sum >= (double)top_p,
 *                    crossing entry included, never empty.
 *   min_p  in (0,1]: prefix of entries with w >= min_p * w[0] (fp32 product).
 * ==================================================================================== */
static size_t prefix_draw(size_t n, const float *w, float top_p, float min_p, struct draw_src *d,
                          struct oracle_draw_info *info) {
    size_t keep = n;
    if (top_p > 0.0f && top_p < 1.0f) {
        double cum = 0.0;
        size_t cut = 0;
        for (cut = 0; cut < n; cut++) {
            cum += (double) w[cut];
            if (cum >= (double) top_p) {
                cut++;
                break;
            }
        }
        if (cut < 1)
            cut = 1;
        keep = cut;
    }
    if (min_p > 0.0f) {
        const float floor_w = min_p * w[0];
        size_t      m       = 0;
        while (m < n && w[m] >= floor_w)
            m++;
        if (m < 1)
            m = 1;
        if (m < keep)
            keep = m;
    }
    double mass = 0.0;
    for (size_t i = 0; i < keep; i++)
        mass += (double) w[i];

    const double target = (double) take_draw(d) * mass;
    double       run    = 0.0;
    size_t       pick   = keep - 1; /* sampler.c:292 */
    double       lo = 0.0, hi = mass;
    int          found = 0;
    for (size_t i = 0; i < keep; i++) {
        const double before = run;
        run += (double) w[i];
        if (target < run) {
            pick  = i;
            lo    = before;
            hi    = run;
            found = 1;
            break;
        }
    }
    if (info) {
        double dist         = found ? fmin(target - lo, hi - target) : 0.0;
        info->boundary_dist = mass > 0.0 ? dist / mass : 0.0;
        info->mass          = mass;
        info->n_keep        = keep;
        info->draws         = d->taken;
    }
    return pick;
}

double oracle_softmax_normalised(size_t n, const float *logits, float temperature, float *pn) {
    const double sum = oracle_softmax_into(n, logits, temperature, pn);
    for (size_t i = 0; i < n; i++)
        pn[i] = (float) ((double) pn[i] / sum); /* sampler.c:251-253 */
    return sum;
}

/* Full-vocabulary path with prefix filters: softmax over all n in index order, normalise,
 * order by probability, then prefix_draw. top_p alone reproduces sampler.c:246-304. */
static int32_t sorted_prob_core(size_t n, const float *logits, float top_p, float min_p,
                                float temperature, struct draw_src *d,
                                struct oracle_draw_info *info) {
    float *pn = (float *) malloc(n * sizeof(float));
    if (!pn) {
        info_none(info);
        return oracle_argmax(n, logits);
    }
    const double sum = oracle_softmax_into(n, logits, temperature, pn);
    if (sum <= 0.0) { /* sampler.c:247-249 */
        free(pn);
        info_none(info);
        return oracle_argmax(n, logits);
    }
    for (size_t i = 0; i < n; i++)
        pn[i] = (float) ((double) pn[i] / sum);
    struct keyed *v = keyed_from(n, pn);
    if (!v || sort_desc(v, n) != 0) {
        free(v);
        free(pn);
        info_none(info);
        return oracle_argmax(n, logits);
    }
    for (size_t i = 0; i < n; i++)
        pn[i] = v[i].key; /* weights in walk order */
    const size_t  at   = prefix_draw(n, pn, top_p, min_p, d, info);
    const int32_t pick = (int32_t) v[at].idx;
    free(v);
    free(pn);
    return pick;
}

/* ======================================================================================
 * top-p (sampler.c:232-305)
 * ==================================================================================== */
static int32_t top_p_core(size_t n, const float *logits, float top_p, float temperature,
                          struct draw_src *d, struct oracle_draw_info *info) {
    if (top_p <= 0.0f || temperature <= 0.0f) {
        info_none(info);
        return oracle_argmax(n, logits);
    }
    if (top_p >= 1.0f)
        return temperature_core(n, logits, temperature, d, info);
    return sorted_prob_core(n, logits, top_p, 0.0f, temperature, d, info);
}

/* ---- public wrappers ------------------------------------------------------------------ */
int32_t oracle_temperature_u(size_t n, const float *l, float t, float u,
                             struct oracle_draw_info *info) {
    struct draw_src d = {NULL, u, 0};
    return temperature_core(n, l, t, &d, info);
}
int32_t oracle_top_k_u(size_t n, const float *l, int k, float t, float u,
                       struct oracle_draw_info *info) {
    struct draw_src d = {NULL, u, 0};
    return top_k_core(n, l, k, t, &d, info);
}
int32_t oracle_top_p_u(size_t n, const float *l, float p, float t, float u,
                       struct oracle_draw_info *info) {
    struct draw_src d = {NULL, u, 0};
    return top_p_core(n, l, p, t, &d, info);
}
int32_t oracle_temperature(size_t n, const float *l, float t, struct oracle_rng *rng) {
    struct draw_src d = {rng, 0.0f, 0};
    return temperature_core(n, l, t, &d, NULL);
}
int32_t oracle_top_k(size_t n, const float *l, int k, float t, struct oracle_rng *rng) {
    struct draw_src d = {rng, 0.0f, 0};
    return top_k_core(n, l, k, t, &d, NULL);
}
int32_t oracle_top_p(size_t n, const float *l, float p, float t, struct oracle_rng *rng) {
    struct draw_src d = {rng, 0.0f, 0};
    return top_p_core(n, l, p, t, &d, NULL);
}

/* ======================================================================================
 * Session sampler state and dispatch.
 * ==================================================================================== */
void oracle_session_defaults(struct oracle_session_sampler *s) {
    /* arch_state.c:1168-1173 */
    s->temperature = 0.0f;
    s->top_p       = 1.0f;
    s->top_k       = 0;
    oracle_rng_seed(&s->rng, UINT64_C(0xCAFEBABE1234));
}

void oracle_session_apply_opts(struct oracle_session_sampler *s, float temperature, float top_p,
                               int top_k, uint64_t random_seed) {
    /* step.c:390-396 */
    s->temperature = temperature;
    s->top_p       = top_p > 0.0f ? top_p : 1.0f;
    s->top_k       = top_k;
    if (random_seed != 0)
        oracle_rng_seed(&s->rng, random_seed);
}

int oracle_session_draws(const struct oracle_session_sampler *s, size_t n) {
    (void) n; /* top_k >= n falls through to the temperature path, which also draws once */
    return s->temperature == 0.0f ? 0 : (s->temperature > 0.0f ? 1 : 0);
}

void oracle_softcap_inplace(size_t n, float *logits, float cap) {
    for (size_t i = 0; i < n; i++)
        logits[i] = tanhf(logits[i] / cap) * cap; /* head.c:153-155 */
}

int32_t oracle_finalize_row(struct oracle_session_sampler *s, size_t n, float *logits,
                            float softcap) {
    /* head.c:148-159: soft-cap only when a stochastic mode will read the values. */
    if (softcap > 0.0f && s->temperature > 0.0f)
        oracle_softcap_inplace(n, logits, softcap);
    /* head.c:172-183 */
    if (s->temperature == 0.0f)
        return oracle_argmax(n, logits);
    if (s->top_k > 1)
        return oracle_top_k(n, logits, s->top_k, s->temperature, &s->rng);
    if (s->top_p > 0.0f && s->top_p < 1.0f)
        return oracle_top_p(n, logits, s->top_p, s->temperature, &s->rng);
    return oracle_temperature(n, logits, s->temperature, &s->rng);
}

void oracle_finalize_batch(struct oracle_session_sampler *s, size_t k, size_t n, float *logits,
                           float softcap, int32_t *out_tokens) {
    /* head.c:274-304: rows in order, one shared RNG. */
    for (size_t r = 0; r < k; r++)
        out_tokens[r] = oracle_finalize_row(s, n, logits + r * n, softcap);
}

/* ======================================================================================
 * Penalties (defined here).
 * ==================================================================================== */
void oracle_apply_penalties(size_t n, float *logits, const int32_t *hist, size_t hist_len,
                            float rep, float freq, float pres) {
    if (!hist || hist_len == 0)
        return;
    uint32_t *cnt = (uint32_t *) calloc(n, sizeof *cnt);
    if (!cnt)
        return;
    for (size_t h = 0; h < hist_len; h++) {
        const int32_t t = hist[h];
        if (t >= 0 && (size_t) t < n)
            cnt[t]++;
    }
    for (size_t i = 0; i < n; i++) {
        if (!cnt[i])
            continue;
        float l = logits[i];
        l       = l > 0.0f ? l / rep : l * rep;
        {
            volatile float prod = freq * (float) cnt[i]; /* keep the product a separate rounding */
            l                   = l - prod;
        }
        l         = l - pres;
        logits[i] = l;
    }
    free(cnt);
}

/* ======================================================================================
 * The chain (defined here; reduces to the reference modes as the header states).
 * ==================================================================================== */
static int32_t chain_core(size_t n, const float *logits, const struct oracle_chain_params *p,
                          struct draw_src *d, struct oracle_draw_info *info) {
    const float T = p->temperature;
    if (T <= 0.0f) {
        info_none(info);
        return oracle_argmax(n, logits);
    }
    const int use_p   = p->top_p > 0.0f && p->top_p < 1.0f;
    const int use_m   = p->min_p > 0.0f;
    const int use_k   = p->top_k > 1 && (size_t) p->top_k < n;
    const float top_p = use_p ? p->top_p : 1.0f;
    const float min_p = use_m ? p->min_p : 0.0f;

    if (!use_k) {
        if (!use_p && !use_m)
            return temperature_core(n, logits, T, d, info);
        return sorted_prob_core(n, logits, top_p, min_p, T, d, info);
    }
    if (!use_p && !use_m)
        return top_k_core(n, logits, p->top_k, T, d, info);

    /* top-k survivors, then the prefix filters on their renormalised probabilities. */
    struct keyed *v = keyed_from(n, logits);
    if (!v || sort_desc(v, n) != 0) {
        free(v);
        info_none(info);
        return oracle_argmax(n, logits);
    }
    size_t k = (size_t) p->top_k;
    if (k > ORACLE_TOPK_CAP)
        k = ORACLE_TOPK_CAP;
    float *kl = (float *) malloc(2 * k * sizeof(float));
    float *kp = kl + k;
    for (size_t j = 0; j < k; j++)
        kl[j] = v[j].key;
    const double sum = oracle_softmax_into(k, kl, T, kp);
    for (size_t j = 0; j < k; j++)
        kp[j] = (float) ((double) kp[j] / sum);
    const size_t  at   = prefix_draw(k, kp, top_p, min_p, d, info);
    const int32_t pick = (int32_t) v[at].idx;
    free(kl);
    free(v);
    return pick;
}

int32_t oracle_sample_chain_u(size_t n, const float *logits, const struct oracle_chain_params *p,
                              float u, struct oracle_draw_info *info) {
    struct draw_src d = {NULL, u, 0};
    return chain_core(n, logits, p, &d, info);
}

/* ======================================================================================
 * Speculative verification (defined here).
 * ==================================================================================== */
int32_t oracle_spec_verify(size_t L, size_t n, const float *target, size_t ld_t, const float *q,
                           size_t ld_q, const int32_t *draft, const float *u, float temperature,
                           int32_t *out_tokens) {
    if (temperature <= 0.0f) {
        size_t j = 0;
        for (; j < L; j++) {
            const int32_t best = oracle_argmax(n, target + j * ld_t);
            if (best != draft[j]) {
                out_tokens[j] = best;
                return (int32_t) j;
            }
            out_tokens[j] = draft[j];
        }
        out_tokens[L] = oracle_argmax(n, target + L * ld_t);
        return (int32_t) L;
    }
    float *pn = (float *) malloc(n * sizeof(float));
    for (size_t j = 0; j < L; j++) {
        const float *row = target + j * ld_t;
        const float *qj  = q + j * ld_q;
        oracle_softmax_normalised(n, row, temperature, pn);
        const int32_t x = draft[j];
        if ((double) u[j] * (double) qj[x] < (double) pn[x]) {
            out_tokens[j] = x;
            continue;
        }
        /* first rejection: resample from the normalised positive part of p - q */
        double R = 0.0;
        for (size_t i = 0; i < n; i++) {
            const float r = pn[i] - qj[i];
            if (r > 0.0f)
                R += (double) r;
        }
        int32_t tok;
        if (R > 0.0) {
            const double tgt  = (double) u[L] * R;
            double       run  = 0.0;
            size_t       last = 0, i;
            int          hit  = 0;
            for (i = 0; i < n; i++) {
                const float r = pn[i] - qj[i];
                if (r > 0.0f) {
                    run += (double) r;
                    last = i;
                    if (tgt < run) {
                        hit = 1;
                        break;
                    }
                }
            }
            tok = (int32_t) (hit ? i : last);
        } else {
            tok = oracle_temperature_u(n, row, temperature, u[L], NULL);
        }
        out_tokens[j] = tok;
        free(pn);
        return (int32_t) j;
    }
    free(pn);
    out_tokens[L] = oracle_temperature_u(n, target + L * ld_t, temperature, u[L], NULL);
    return (int32_t) L;
}

/* ======================================================================================
 * Row-parallel helpers for the CPU timing leg: one row per thread, the reference's own
 * concurrency model (one thread per session, include/geist_arch.h:43-51).
 * ==================================================================================== */
int oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void oracle_batch_top_k_u(size_t rows, size_t n, const float *logits, size_t ld, int top_k,
                          float temperature, const float *u, int32_t *out, int threads) {
    if (threads < 1)
        threads = 1;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
    for (long r = 0; r < (long) rows; r++)
        out[r] = oracle_top_k_u(n, logits + (size_t) r * ld, top_k, temperature, u[r], NULL);
}

void oracle_batch_chain_u(size_t rows, size_t n, const float *logits, size_t ld,
                          const struct oracle_chain_params *p, const int32_t *hist, size_t hist_ld,
                          const int32_t *hist_len, float rep, float freq, float pres,
                          const float *u, int32_t *out, int threads) {
    if (threads < 1)
        threads = 1;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
    for (long r = 0; r < (long) rows; r++) {
        const float *row = logits + (size_t) r * ld;
        float       *tmp = NULL;
        if (hist && hist_len && hist_len[r] > 0) {
            tmp = (float *) malloc(n * sizeof(float));
            memcpy(tmp, row, n * sizeof(float));
            oracle_apply_penalties(n, tmp, hist + (size_t) r * hist_ld, (size_t) hist_len[r], rep,
                                   freq, pres);
            row = tmp;
        }
        out[r] = oracle_sample_chain_u(n, row, p, u[r], NULL);
        free(tmp);
    }
}

/* tools/eval_geist.c:63-73 */
double oracle_logprob_at(size_t n, const float *logits, int32_t token) {
    float maxv = logits[0];
    for (size_t i = 1; i < n; i++)
        if (logits[i] > maxv)
            maxv = logits[i];
    double sum = 0.0;
    for (size_t i = 0; i < n; i++)
        sum += exp((double) (logits[i] - maxv));
    return (double) (logits[token] - maxv) - log(sum);
}

/* src/engine/session.c:437-513. Lengths are tried longest first; for one length the history is
 * walked from the most recent start position backwards, a later find only replaces an earlier
 * one when more tokens follow it, and the walk stops once k_max - 1 follow. */
size_t oracle_propose_drafts_ngram(const int32_t *history, size_t n, int32_t seed, size_t k_max,
                                   size_t max_suffix, int32_t *out, size_t *match_len) {
    out[0] = seed;
    if (match_len)
        *match_len = 0;
    if (k_max <= 1 || n == 0)
        return 1;
    const size_t want = k_max - 1;
    for (size_t len = max_suffix > 8 ? 8 : max_suffix; len >= 1; len--) {
        const size_t ctx = len - 1; /* history tokens in the suffix; the seed is its last */
        if (ctx > n)
            continue;
        const int32_t *tail  = history + (n - ctx);
        bool           have  = false;
        size_t         at    = 0, gain = 0;
        for (size_t start = n - ctx; start-- > 0;) {
            if (ctx && memcmp(history + start, tail, ctx * sizeof *history) != 0)
                continue;
            if (history[start + ctx] != seed)
                continue;
            const size_t next = start + len;
            if (next >= n)
                continue; /* nothing follows */
            const size_t room = n - next < want ? n - next : want;
            if (!have || room > gain) {
                have = true;
                at   = start;
                gain = room;
                if (gain >= want)
                    break;
            }
        }
        if (have) {
            memcpy(out + 1, history + at + len, gain * sizeof *out);
            if (match_len)
                *match_len = len;
            return 1 + gain;
        }
    }
    return 1;
}
