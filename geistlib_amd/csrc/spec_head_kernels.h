/* Launchers of the speculative output head (spec_head.hip): the reference's greedy-only
 * sketch head (src/archs/transformer/forward/spec_head.c) for a tied F16 table in device
 * memory. */
#ifndef GEIST_SPEC_HEAD_KERNELS_H
#define GEIST_SPEC_HEAD_KERNELS_H

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace gs {

/* Scalars of one call, in device memory. */
struct SpecScalars {
    float inv_xq;     /* max|h| / 127 */
    float h_l1_kept;  /* L1 norm of h over the kept dimensions */
    float h_l2_drop;  /* L2 norm of h over the dropped dimensions */
    float threshold;  /* a lower bound of the topk-th largest group maximum: the topk best rows are >= it */
    float cutoff;     /* the topk-th largest rough score */
    int   n_cand;     /* rows >= threshold */
    int   n_final;    /* topk, or 0 when the candidates did not fit the list */
};

/* What a call answers (mirrors struct geist_hip_spec_result). */
struct SpecResult {
    int32_t token;
    int32_t answered;
    int32_t n_finalists;
    int32_t n_listed;
    float   cutoff;
    float   best_exact;
};

struct SpecHeadDev {
    long vocab;
    int  d_model, sketch_dim, topk;
    int  n_groups; /* ceil(vocab / 32): groups of consecutive rows whose maximum the projection leaves */
    int  list_cap; /* 2 topk candidates */
    const uint16_t *w; /* [vocab, d_model] binary16, not owned */
    /* built once */
    int8_t   *sketch;    /* [vocab, sketch_dim] */
    float    *row_scale; /* [vocab] */
    float    *w_drop;    /* [vocab] */
    float    *w_l1;      /* [vocab] */
    uint32_t *dims;      /* [sketch_dim] ascending */
    uint8_t  *kept;      /* [d_model] 1 where the sketch keeps the dimension */
    /* per call */
    float       *act;   /* [sketch_dim] the kept dimensions of the int8 activation, as floats */
    float       *rough; /* [vocab], allocated up to a multiple of 32 */
    float       *gmax;  /* [n_groups] maxima of the rough scores of 32 consecutive rows */
    SpecScalars *sc;
    int32_t     *fin_idx;    /* [topk] the finalists, any order */
    float       *fin_exact;  /* [topk] their exact logits */
};

/* The selection kernels hold their keys in registers, 1024 threads: up to 32 group maxima each
 * (a vocabulary of 2^20 rows) and up to 8 candidates each (2 x 4096). */
constexpr int SPEC_TMAX_EPT_MAX = 32;
constexpr int SPEC_LIST_EPT_MAX = 8;
constexpr int SPEC_VOCAB_MAX    = SPEC_TMAX_EPT_MAX * 1024 * 32;
constexpr int SPEC_TOPK_MAX     = 4096;
/* Largest d_model the finalist kernel stages in LDS. */
constexpr int SPEC_D_MODEL_MAX = 5120;
/* The rough scores are sums of products of two int8 values (|v| <= 127) formed in binary32:
 * exact while sketch_dim * 127 * 127 < 2^24. */
constexpr int SPEC_SKETCH_DIM_MAX = 1040;

/* dvar[i] = variance of dimension i over the rows 0, vstep, 2 vstep, ... (spec_head.c:505-522,
 * binary32, rows in order). */
void launch_spec_dim_stats(hipStream_t stream, const uint16_t *w, long vocab, int d_model,
                           long vstep, float *dvar);
/* sketch, row_scale, w_drop, w_l1 from w, dims and kept (spec_head.c:563-603). */
void launch_spec_sketch_rows(hipStream_t stream, const SpecHeadDev &d);
/* transformer_spec_head_try for one normed hidden row h [d_model] (spec_head.c:624-889). With
 * norm_w != NULL, h is the hidden row before the output norm: the norm (weights norm_w, eps) runs
 * in the first kernel and h_normed [d_model] receives the normed row. */
void launch_spec_try(hipStream_t stream, const SpecHeadDev &d, const float *h, bool verify,
                     SpecResult *result, const float *norm_w = nullptr, float eps = 0.0f,
                     float *h_normed = nullptr);

} // namespace gs
#endif
