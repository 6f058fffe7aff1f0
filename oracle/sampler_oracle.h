/*
 * sampler_oracle.h -- CPU restatement of the reference token sampler.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing in the shipped library links, loads or calls this
 * code: it exists so that tests, the smoke check and the cpu_baseline leg of the
 * benchmark can compare the HIP path against the reference algorithm.
 *
 * Every function names the reference lines it follows (paths relative to the reference
 * tree). Stages the reference does not have (penalties, min-p, the top-k -> top-p ->
 * min-p chain, speculative rejection sampling) are DEFINED here; their parity is pinned
 * by closed forms and brute force in tests/, not by the reference.
 *
 * Third-party arithmetic on this path: libm expf/tanhf and libc qsort (glibc 2.35).
 * The reference's ordering of equal keys is whatever qsort does with a comparator
 * that returns 0 (src/engine/sampler.c:167-176); glibc 2.35's qsort is a stable merge
 * sort, so equal keys keep ascending index order. This restatement fixes that order by
 * definition (key descending, index ascending). NaN logits make the reference
 * comparator non-transitive; here NaN sorts after every number ("parity unpinned"
 * for rows that contain NaN in top-k / top-p mode).
 */
#ifndef GEIST_SAMPLER_ORACLE_H
#define GEIST_SAMPLER_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- RNG: src/engine/sampler.h:28-32, sampler.c:27-48 ------------------------------ */
struct oracle_rng {
    uint64_t state;
};
void     oracle_rng_seed(struct oracle_rng *rng, uint64_t seed);
uint64_t oracle_rng_next_u64(struct oracle_rng *rng);
float    oracle_rng_next_unit(struct oracle_rng *rng);

/* ---- building blocks: sampler.c:52-102 -------------------------------------------- */
int32_t oracle_argmax(size_t n, const float *logits);
double  oracle_softmax_into(size_t n, const float *logits, float temperature, float *probs);

/* Diagnostics every *_u entry point can fill (pass NULL to skip).
 *   boundary_dist: distance of the scaled draw to the nearer edge of the chosen CDF
 *                  slot, divided by the total mass of the walk (so it is comparable
 *                  with the "within 1e-6 of a CDF boundary" rule); +inf when no draw
 *                  was consumed.
 *   n_keep:        number of entries the final walk ran over.
 *   mass:          the double sum the draw was scaled by.                              */
struct oracle_draw_info {
    double boundary_dist;
    double mass;
    size_t n_keep;
    int    draws; /* uniforms consumed: 0 or 1 */
};

/* ---- the four reference modes with the uniform passed in (draw = next_unit value) -- */
int32_t oracle_temperature_u(size_t n, const float *logits, float temperature, float u,
                             struct oracle_draw_info *info);                /* sampler.c:106-132 */
int32_t oracle_top_k_u(size_t n, const float *logits, int top_k, float temperature, float u,
                       struct oracle_draw_info *info);                      /* sampler.c:178-228 */
int32_t oracle_top_p_u(size_t n, const float *logits, float top_p, float temperature, float u,
                       struct oracle_draw_info *info);                      /* sampler.c:232-305 */

/* ---- the same with a caller-owned RNG, consuming draws exactly as the reference ---- */
int32_t oracle_temperature(size_t n, const float *logits, float temperature,
                           struct oracle_rng *rng);
int32_t oracle_top_k(size_t n, const float *logits, int top_k, float temperature,
                     struct oracle_rng *rng);
int32_t oracle_top_p(size_t n, const float *logits, float top_p, float temperature,
                     struct oracle_rng *rng);

/* ---- session sampler state and dispatch -------------------------------------------- */
/* src/archs/transformer/arch_state.c:1168-1173 (defaults),
 * src/archs/transformer/forward/step.c:385-411 (opts), head.c:148-186, 274-304 (dispatch) */
struct oracle_session_sampler {
    float             temperature;
    float             top_p;
    int               top_k;
    struct oracle_rng rng;
};
void    oracle_session_defaults(struct oracle_session_sampler *s);
void    oracle_session_apply_opts(struct oracle_session_sampler *s, float temperature,
                                  float top_p, int top_k, uint64_t random_seed);
/* Whether the dispatch draws one uniform for this configuration (else zero). */
int     oracle_session_draws(const struct oracle_session_sampler *s, size_t n);
void    oracle_softcap_inplace(size_t n, float *logits, float cap);     /* head.c:150-156 */
/* One row: softcap in place iff cap > 0 and T > 0, then the four-way dispatch. */
int32_t oracle_finalize_row(struct oracle_session_sampler *s, size_t n, float *logits,
                            float softcap);
/* k rows, contiguous with row stride n, sequential with one shared RNG. */
void    oracle_finalize_batch(struct oracle_session_sampler *s, size_t k, size_t n,
                              float *logits, float softcap, int32_t *out_tokens);

/* ---- stages defined by this repository (no reference counterpart) ------------------ */
/* Penalties over one row, in place. For every DISTINCT id t in hist[0..hist_len) with
 * 0 <= t < n and c = its number of occurrences:
 *     l = logits[t];  l = l > 0 ? l / rep : l * rep;  l = l - freq * (float)c;  l = l - pres;
 * (repetition as in CTRL / HF, frequency and presence as in the OpenAI API; each step is
 * one fp32 rounding, no fused multiply-add). Ids outside [0, n) are ignored. */
void oracle_apply_penalties(size_t n, float *logits, const int32_t *hist, size_t hist_len,
                            float rep, float freq, float pres);

struct oracle_chain_params {
    float temperature;
    int   top_k;
    float top_p;
    float min_p;
};
/* The sampling chain on one (already penalised, already soft-capped) row:
 *   T <= 0                              -> argmax, no draw.
 *   1 < top_k < n                       -> keep the top_k (value desc, index asc; at most 8192),
 *                                          softmax over them in that order (sampler.c:209-219).
 *   otherwise                           -> softmax over all n in index order; if neither
 *                                          top_p in (0,1) nor min_p in (0,1] is set this is
 *                                          oracle_temperature_u. Else normalise and sort by
 *                                          probability (desc, index asc) as sampler.c:250-270.
 *   top_p in (0,1) or min_p in (0,1]    -> pn_j = (float)((double)p_j / sum); the nucleus is the
 *                                          shortest prefix with cumulative pn >= top_p (inclusive,
 *                                          at least 1; sampler.c:273-283); the min-p prefix is
 *                                          {j : pn_j >= min_p * pn_0} (fp32 product); keep the
 *                                          shorter prefix; draw u * (double sum of kept weights)
 *                                          over the kept prefix in its order (sampler.c:286-299).
 * With only top_k set it equals oracle_top_k_u; with only top_p set, oracle_top_p_u. */
int32_t oracle_sample_chain_u(size_t n, const float *logits, const struct oracle_chain_params *p,
                              float u, struct oracle_draw_info *info);

/* Normalised probabilities of the whole row, pn_i = (float)((double)p_i / sum) with
 * p_i, sum from oracle_softmax_into (sampler.c:246-253). Returns the double sum. */
double oracle_softmax_normalised(size_t n, const float *logits, float temperature, float *pn);

/* Speculative-decode verification of one sequence (Leviathan et al. 2023, Chen et al. 2023).
 *   target: (L+1) rows of n logits, row stride ld_t;  q: L rows of draft probabilities, stride ld_q
 *   draft[L] token ids; u[L+1] uniforms (u[j] tests position j, u[L] draws the last token).
 * T > 0:  pn_j = normalised softmax of target row j. Position j is accepted iff
 *         (double)u[j] * (double)q_j[x_j] < (double)pn_j[x_j]  (u < min(1, p/q), exact in double).
 *         At the first rejected j: r_i = max(0, pn_j[i] - q_j[i]) in fp32, R = double sum in index
 *         order; the emitted token is the first i with (double)u[L]*R < running sum (if R <= 0,
 *         a temperature draw from row j with u[L]). If all L are accepted the bonus token is
 *         oracle_temperature_u(row L, u[L]).
 * T <= 0: position j is accepted iff draft[j] == argmax(row j); the emitted token is the argmax of
 *         the first mismatching row, or of row L (the exact-match loop of src/engine/session.c:599-625).
 * Writes out_tokens[0..n_acc) = draft[0..n_acc), out_tokens[n_acc] = the emitted token and
 * returns n_acc (0..L). */
int32_t oracle_spec_verify(size_t L, size_t n, const float *target, size_t ld_t, const float *q,
                           size_t ld_q, const int32_t *draft, const float *u, float temperature,
                           int32_t *out_tokens);

/* ---- batch helpers used by the cpu_baseline timing leg (OpenMP over rows) ---------- */
void oracle_batch_top_k_u(size_t rows, size_t n, const float *logits, size_t ld, int top_k,
                          float temperature, const float *u, int32_t *out, int threads);
void oracle_batch_chain_u(size_t rows, size_t n, const float *logits, size_t ld,
                          const struct oracle_chain_params *p, const int32_t *hist, size_t hist_ld,
                          const int32_t *hist_len, float rep, float freq, float pres,
                          const float *u, int32_t *out, int threads);
int  oracle_max_threads(void);

/* log_softmax(logits)[token] as the reference's evaluation tool computes it from peeked
 * logits (tools/eval_geist.c:63-73): fp32 max, double exp of the fp32 difference, sequential
 * double sum, (double)(logits[token] - max) - log(sum). */
double oracle_logprob_at(size_t n, const float *logits, int32_t token);

/* The n-gram drafter of the speculative loop (propose_drafts_ngram,
 * src/engine/session.c:437-513): out[0] = seed; then, for the longest suffix of history + [seed]
 * (at most min(max_suffix, 8) tokens) found earlier in the history, the up to k_max - 1 tokens
 * that followed its best occurrence (most following tokens, most recent among equals). Returns
 * the number of drafts (>= 1); *match_len = length of the matched suffix or 0. `out` holds
 * k_max entries. Pinned by a brute-force enumeration over (length, position) in the tests and
 * by worked examples; the reference holds no test of this function. */
size_t oracle_propose_drafts_ngram(const int32_t *history, size_t n, int32_t seed, size_t k_max,
                                   size_t max_suffix, int32_t *out, size_t *match_len);

#ifdef __cplusplus
}
#endif
#endif
