/*
 * spec_head_oracle.h -- TEST INFRASTRUCTURE, not part of the shipped library: a scalar CPU
 * restatement of the reference's speculative output head for greedy decoding
 * (src/archs/transformer/forward/spec_head.c) over a tied F16 table. Only tests/, the smoke check
 * and the cpu_baseline leg of bench.py may load it.
 *
 * The reference's file needs the arch state, the backend tables and OpenMP and does not compile
 * on its own; its test (tests/test_spec_head_sampling_int.c) needs a model file. Pinned instead
 * by what the construction fixes (tests/test_spec_head_oracle.py):
 *   - the contract of that test: whenever the head answers, the token is the dense head's argmax
 *     (dense = oracle_f16_gemv_m1, itself pinned to the compiled reference), on random tables
 *     and on tables built to make the sketch misrank (near-ties, weight hidden in the dropped
 *     dimensions); with the bound switched off such tables do produce a wrong token, so the
 *     check can fail;
 *   - the kept dimensions against a numpy ranking of the sampled variances; sketch values and
 *     row scales against numpy (rint, maximum); the two norms of the bound against float64;
 *   - the integer dot and the top-K selection against numpy (sorted scores);
 *   - the bound itself: for every row, exact logit <= upper bound, checked in float64.
 */
#ifndef GEIST_SPEC_HEAD_ORACLE_H
#define GEIST_SPEC_HEAD_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

struct oracle_spec_head {
    size_t    vocab, d_model, sketch_dim, topk;
    uint32_t *dims;      /* [sketch_dim] kept dimensions, ascending */
    int8_t   *sketch;    /* [vocab, sketch_dim] */
    float    *row_scale; /* [vocab] max|kept w| / 127 */
    float    *w_drop;    /* [vocab] L2 norm of the dropped dimensions */
    float    *w_l1;      /* [vocab] L1 norm of the kept dimensions */
};

/* Geometry of spec_head_build (spec_head.c:402-445): sketch width d_model / stride with stride =
 * d_model / 640 lowered until it divides d_model (stride_override > 0 replaces the default, as
 * GEIST_SPEC_STRIDE does), finalists 1024 or, from 200000 tokens on, 4096 (topk_override > 0 as
 * GEIST_SPEC_TOPK, clamped to 16..vocab). Returns 0 and fills the two sizes when a sketch is
 * built: vocab >= 8192 and 2 * d_model / sketch_dim >= 3. */
int oracle_spec_head_geometry(size_t vocab, size_t d_model, size_t stride_override,
                              size_t topk_override, size_t *sketch_dim, size_t *topk);

/* spec_head_build (spec_head.c:402-607). Returns NULL where the reference declines. */
struct oracle_spec_head *oracle_spec_head_build(const uint16_t *w_f16, size_t vocab, size_t d_model,
                                                size_t stride_override, size_t topk_override);
void                     oracle_spec_head_free(struct oracle_spec_head *sh);

/* transformer_spec_head_try (spec_head.c:624-889) for one normed hidden row, finalists scored
 * with f16_gemv_m1's arithmetic (the reference's x86 route, spec_head.c:787-800). Returns 1 and
 * the token when the bound certifies it, 0 when the head declines (the caller then runs the
 * dense head). With verify == 0 the bound is skipped (GEIST_SPEC_VERIFY=0). rough, if not NULL,
 * receives the vocab rough scores; n_finalists and cutoff what phase 2 kept. */
int oracle_spec_head_try(const struct oracle_spec_head *sh, const uint16_t *w_f16, const float *h,
                         int verify, int32_t *out_token, float *rough, size_t *n_finalists,
                         float *cutoff);

#ifdef __cplusplus
}
#endif
#endif
