/* spec_head_oracle.c -- TEST INFRASTRUCTURE (see spec_head_oracle.h). Scalar restatement of
 * src/archs/transformer/forward/spec_head.c for a tied F16 table. */
#include "spec_head_oracle.h"

#include "lm_head_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#define SKETCH_DIMS_TARGET 640 /* spec_head.c:88 */
#define MIN_ROW_SHRINK 3.0     /* spec_head.c:112 */
#define TOPK_DEFAULT 1024      /* spec_head.c:119 */

static size_t clamp_sz(size_t v, size_t lo, size_t hi) { return v < lo ? lo : (v > hi ? hi : v); }

int oracle_spec_head_geometry(size_t vocab, size_t d_model, size_t stride_override,
                              size_t topk_override, size_t *sketch_dim, size_t *topk) {
    /* spec_head.c:431-448 */
    const size_t stride_dflt = d_model > SKETCH_DIMS_TARGET ? d_model / SKETCH_DIMS_TARGET : 1;
    size_t       sub = stride_override ? clamp_sz(stride_override, 1, d_model) : stride_dflt;
    while (sub > 1 && d_model % sub != 0)
        sub--;
    const size_t topk_dflt = vocab >= 200000 ? 4096 : TOPK_DEFAULT;
    const size_t k         = topk_override ? clamp_sz(topk_override, 16, vocab) : topk_dflt;
    if (vocab < 8192)
        return -1;
    const size_t sd = d_model / sub;
    if ((double) (2 * d_model) / (double) sd < MIN_ROW_SHRINK)
        return -1;
    *sketch_dim = sd;
    *topk       = k;
    return 0;
}

static void row_to_f32(const uint16_t *row, size_t n, float *dst) {
    for (size_t i = 0; i < n; i++)
        dst[i] = oracle_f16_to_f32(row[i]);
}

void oracle_spec_head_free(struct oracle_spec_head *sh) {
    if (!sh)
        return;
    free(sh->dims);
    free(sh->sketch);
    free(sh->row_scale);
    free(sh->w_drop);
    free(sh->w_l1);
    free(sh);
}

struct oracle_spec_head *oracle_spec_head_build(const uint16_t *w, size_t V, size_t H,
                                                size_t stride_override, size_t topk_override) {
    size_t SD, topk;
    if (oracle_spec_head_geometry(V, H, stride_override, topk_override, &SD, &topk) != 0)
        return NULL;
    struct oracle_spec_head *sh = calloc(1, sizeof *sh);
    sh->vocab = V, sh->d_model = H, sh->sketch_dim = SD, sh->topk = topk;
    sh->dims      = malloc(SD * sizeof(uint32_t));
    sh->sketch    = malloc(V * SD);
    sh->row_scale = malloc(V * sizeof(float));
    sh->w_drop    = malloc(V * sizeof(float));
    sh->w_l1      = malloc(V * sizeof(float));
    float *tmp    = malloc(H * sizeof(float));
    float *dvar   = calloc(H, sizeof(float));
    float *dsum   = calloc(H, sizeof(float));
    char  *kept   = calloc(H, 1);

    /* spec_head.c:505-522: per-dimension variance over every vstep-th row */
    const size_t vstep = V > 512 ? V / 512 : 1;
    size_t       vn    = 0;
    for (size_t r = 0; r < V; r += vstep, vn++) {
        row_to_f32(w + r * H, H, tmp);
        for (size_t i = 0; i < H; i++) {
            dsum[i] += tmp[i];
            dvar[i] += tmp[i] * tmp[i];
        }
    }
    for (size_t i = 0; i < H; i++) {
        const float mean = dsum[i] / (float) vn;
        dvar[i]          = dvar[i] / (float) vn - mean * mean;
    }
    /* spec_head.c:526-536: the SD largest, the first of equals */
    for (size_t s = 0; s < SD; s++) {
        size_t best = 0;
        for (size_t i = 1; i < H; i++)
            if (dvar[i] > dvar[best])
                best = i;
        sh->dims[s] = (uint32_t) best;
        dvar[best]  = -1.0f;
    }
    /* spec_head.c:540-548: ascending */
    for (size_t a = 0; a + 1 < SD; a++)
        for (size_t b = a + 1; b < SD; b++)
            if (sh->dims[b] < sh->dims[a]) {
                const uint32_t t = sh->dims[a];
                sh->dims[a]      = sh->dims[b];
                sh->dims[b]      = t;
            }
    for (size_t s = 0; s < SD; s++)
        kept[sh->dims[s]] = 1;

    /* spec_head.c:563-603 (rows are independent; the reference runs them in parallel too) */
#pragma omp parallel for schedule(static)
    for (size_t r = 0; r < V; r++) {
        float tmp[H];
        row_to_f32(w + r * H, H, tmp);
        float amax = 1e-8f;
        for (size_t s = 0; s < SD; s++) {
            const float a = fabsf(tmp[sh->dims[s]]);
            if (a > amax)
                amax = a;
        }
        const float scale = 127.0f / amax;
        int8_t     *sk    = sh->sketch + r * SD;
        for (size_t s = 0; s < SD; s++) {
            long q = lrintf(tmp[sh->dims[s]] * scale);
            q      = q > 127 ? 127 : (q < -127 ? -127 : q);
            sk[s]  = (int8_t) q;
        }
        sh->row_scale[r] = amax / 127.0f;
        float sq = 0.0f, l1 = 0.0f;
        for (size_t i = 0; i < H; i++) {
            if (kept[i])
                l1 += fabsf(tmp[i]);
            else
                sq += tmp[i] * tmp[i];
        }
        sh->w_drop[r] = sqrtf(sq);
        sh->w_l1[r]   = l1;
    }
    free(tmp), free(dvar), free(dsum), free(kept);
    return sh;
}

struct cand {
    float    s;
    uint32_t idx;
};

int oracle_spec_head_try(const struct oracle_spec_head *sh, const uint16_t *w, const float *h,
                         int verify, int32_t *out_token, float *rough_out, size_t *n_finalists,
                         float *cutoff_out) {
    const size_t H = sh->d_model, V = sh->vocab, SD = sh->sketch_dim, topk = sh->topk;
    int8_t      *x_i8  = malloc(H);
    int8_t      *a_sk  = malloc(SD);
    float       *rough = malloc(V * sizeof(float));
    struct cand *heap  = malloc(topk * sizeof *heap);

    /* spec_head.c:672-694: the activation in int8, then its kept dimensions */
    float amax = 1e-8f;
    for (size_t i = 0; i < H; i++) {
        const float a = h[i] < 0.0f ? -h[i] : h[i];
        if (a > amax)
            amax = a;
    }
    const float x_q = 127.0f / amax;
    for (size_t i = 0; i < H; i++) {
        long q  = lrintf(h[i] * x_q);
        q       = q > 127 ? 127 : (q < -127 ? -127 : q);
        x_i8[i] = (int8_t) q;
    }
    for (size_t s = 0; s < SD; s++)
        a_sk[s] = x_i8[sh->dims[s]];

    /* spec_head.c:698-708: rough scores */
#pragma omp parallel for schedule(static)
    for (size_t r = 0; r < V; r++) {
        int32_t       d  = 0;
        const int8_t *sk = sh->sketch + r * SD;
        for (size_t s = 0; s < SD; s++)
            d += (int32_t) a_sk[s] * (int32_t) sk[s];
        rough[r] = (float) d * sh->row_scale[r];
    }

    /* spec_head.c:712-724: activation halves of the bound */
    float h_l1_kept = 0.0f, h_sq_drop = 0.0f;
    for (size_t i = 0; i < H; i++)
        h_sq_drop += h[i] * h[i];
    for (size_t s = 0; s < SD; s++) {
        const float hv = h[sh->dims[s]];
        h_l1_kept += hv < 0.0f ? -hv : hv;
        h_sq_drop -= hv * hv;
    }
    if (h_sq_drop < 0.0f)
        h_sq_drop = 0.0f;
    const float h_l2_drop = sqrtf(h_sq_drop);

    /* spec_head.c:728-770: bounded min-heap of the topk best rough scores */
    size_t hn = 0;
    for (size_t r = 0; r < V; r++) {
        const float sc = rough[r];
        if (hn < topk) {
            size_t i    = hn++;
            heap[i].s   = sc;
            heap[i].idx = (uint32_t) r;
            while (i > 0) {
                const size_t p = (i - 1) >> 1;
                if (heap[p].s <= heap[i].s)
                    break;
                const struct cand t = heap[p];
                heap[p]             = heap[i];
                heap[i]             = t;
                i                   = p;
            }
        } else if (sc > heap[0].s) {
            heap[0].s   = sc;
            heap[0].idx = (uint32_t) r;
            size_t i    = 0;
            for (;;) {
                const size_t l = 2 * i + 1, rg = 2 * i + 2;
                size_t       sm = i;
                if (l < topk && heap[l].s < heap[sm].s)
                    sm = l;
                if (rg < topk && heap[rg].s < heap[sm].s)
                    sm = rg;
                if (sm == i)
                    break;
                const struct cand t = heap[sm];
                heap[sm]            = heap[i];
                heap[i]             = t;
                i                   = sm;
            }
        }
    }

    /* spec_head.c:802-826: exact logits of the finalists (x86 route: the dense kernel's row
     * loop), everything else -inf, argmax with the lowest index among equals */
    int32_t best     = 0;
    float   best_val = -INFINITY;
    int     have     = 0;
    for (size_t c = 0; c < hn; c++) {
        float y;
        oracle_f16_gemv_m1(1, H, h, w + (size_t) heap[c].idx * H, &y);
        if (!have || y > best_val || (y == best_val && (int32_t) heap[c].idx < best)) {
            best     = (int32_t) heap[c].idx;
            best_val = y;
            have     = 1;
        }
    }
    *out_token = best;

    /* spec_head.c:846-872: could an excluded row have won? */
    const float cutoff = hn > 0 ? heap[0].s : -3.4e38f;
    const float inv_xq = 1.0f / x_q;
    int         certain = 1;
    if (verify) {
        for (size_t r = 0; r < V; r++) {
            if (rough[r] > cutoff)
                continue;
            const float ub = rough[r] * inv_xq + 0.5f * sh->row_scale[r] * h_l1_kept +
                             0.5f * sh->w_l1[r] * inv_xq + sh->w_drop[r] * h_l2_drop;
            if (ub > best_val) {
                certain = 0;
                break;
            }
        }
    }
    if (rough_out)
        memcpy(rough_out, rough, V * sizeof(float));
    if (n_finalists)
        *n_finalists = hn;
    if (cutoff_out)
        *cutoff_out = cutoff;
    free(x_i8), free(a_sk), free(rough), free(heap);
    return certain;
}
