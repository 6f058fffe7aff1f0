/*
 * geist_head_hip.h -- the sampler side of the reference's output head, for logits that stay on
 * the device. Mirrors, function for function, what src/archs/transformer/forward/head.c and
 * step.c do between "the lm_head wrote [k, vocab] logits into scratch_logits" and "token ids":
 *
 *   geist_hip_head_create          sampler defaults of transformer_session_alloc
 *                                  (src/archs/transformer/arch_state.c:1168-1173)
 *   geist_hip_head_apply_opts      transformer_session_apply_opts (forward/step.c:385-411)
 *   geist_hip_head_finalize_one_row   sampler part of finalize_logits_one_row (head.c:131-188)
 *   geist_hip_head_finalize_batch     sampler part of finalize_logits_batch (head.c:274-304)
 *   geist_hip_head_argmax_f32      the backend slot fused->argmax_f32
 *                                  (include/geist_backend.h:414-421)
 *   geist_hip_head_project_finalize  output norm + tied F16 lm_head + the above, logits never
 *                                  on the host (head.c:94-188, 224-304)
 *   geist_hip_head_project_finalize_q8w  the same with the int8 table of the x86 backend
 *                                  (src/backends/cpu_x86/backend.c:332-372)
 *   geist_hip_head_spec_build, geist_hip_head_project_finalize_spec  the speculative int8
 *                                  sketch head of greedy decoding (forward/spec_head.c)
 *   geist_hip_head_propose_drafts  the n-gram drafter of geist_session_decode_speculative
 *                                  (src/engine/session.c:437-513, 564-572)
 *   geist_hip_head_spec_accept     the accept loop of geist_session_decode_speculative
 *                                  (src/engine/session.c:599-625) over the rows verify_forward
 *                                  produced (src/archs/transformer/arch_ops.c:176-270)
 *
 * The RNG state of the session lives in device memory and advances there, one draw per
 * stochastic row in row order, exactly as the reference's single host RNG does.
 */
#ifndef GEIST_HEAD_HIP_H
#define GEIST_HEAD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef GEIST_VERSION_MAJOR /* the reference's <geist.h> is not in this translation unit */
/* Layout of struct geist_session_opts, include/geist.h:209-247. */
struct geist_session_opts {
    size_t      max_seq_len;
    float       temperature;
    float       top_p;
    int         top_k;
    uint64_t    random_seed;
    const char *awq_scales_path;
    int         kv_mode; /* enum geist_kv_mode */
    size_t      m_max;
};
#endif

struct geist_hip_head;

/* `vocab` logits per row, at most `m_max` rows per batch call (0 = 64, the reference's default,
 * include/geist.h:244-246). `logit_softcap` is the model's soft-cap (0 = none), applied only
 * when temperature > 0 (head.c:148-149). Returns a geist_status value. */
int geist_hip_head_create(int device, size_t vocab, size_t m_max, float logit_softcap,
                          void *stream, struct geist_hip_head **out);
void geist_hip_head_destroy(struct geist_hip_head *h);
const char *geist_hip_head_errmsg(const struct geist_hip_head *h);

/* opts == NULL keeps the greedy defaults (geist_session_create's NULL opts). Sizes the sampler's
 * workspace for the options it sets, as step.c:398-409 does, so that no later call allocates. */
int geist_hip_head_apply_opts(struct geist_hip_head *h, const struct geist_session_opts *opts);
/* Sizes what geist_hip_head_project_finalize[_q8w|_spec] need for hidden rows of d_model floats:
 * the [m_max, vocab] logit buffer, the normed rows and the scratch of the batch projection
 * (where the reference's session allocator sizes scratch_logits and scratch_normed,
 * src/archs/transformer/arch_state.c). Call it at set-up; a projection call for which nothing
 * was reserved reserves on its first use. */
int geist_hip_head_reserve_projection(struct geist_hip_head *h, size_t d_model);

/* d_logits: [1, vocab] / [k, vocab] fp32 in device memory, row stride vocab. Synchronous: the
 * token ids are in host memory on return, as in the reference. */
int geist_hip_head_finalize_one_row(struct geist_hip_head *h, const float *d_logits,
                                    int32_t *out_token);
int geist_hip_head_finalize_batch(struct geist_hip_head *h, const float *d_logits, size_t k,
                                  int32_t *out_tokens);
int geist_hip_head_argmax_f32(struct geist_hip_head *h, const float *d_logits, size_t n,
                              int32_t *out_index);

/* The whole tail of a forward pass for k <= m_max rows of final hidden states, on the device
 * (head.c:94-188 for one row, 224-304 for a batch): RMS norm with the output-norm weight
 * (head.c:99-101), the tied F16 lm_head (head.c:114-126; [vocab, d_model] binary16, row-major,
 * 16-byte aligned, d_model a multiple of 8), the soft-cap and the session's sampler. The logits
 * live in a buffer of the head and are never copied out; they equal, bit for bit, what the
 * reference's cpu_scalar_rmsnorm and its x86 backend's projection produce -- f16_gemv_m1 for
 * k == 1, the portable cpu_scalar_w_quant_mN (double accumulation) for k > 1, which is what that
 * backend runs for a batch -- so the tokens are those of geist_hip_head_finalize_batch on the
 * reference's logits. Row r of d_hidden starts at
 * d_hidden + r * ld_hidden and is left untouched. */
int geist_hip_head_project_finalize(struct geist_hip_head *h, const float *d_hidden,
                                    size_t ld_hidden, size_t k, const float *d_norm_weight,
                                    float rms_eps, const uint16_t *d_embed_f16, size_t d_model,
                                    int32_t *out_tokens);
/* GEIST_HIP_PROJECTION_X86 (default), _PORTABLE or _X86_AVX2 (include/geist_lm_head_hip.h): which
 * backend's arithmetic the project_finalize calls use. */
int geist_hip_head_set_projection(struct geist_hip_head *h, int mode);
/* GEIST_HIP_SUMS_EXACT (default) or GEIST_HIP_SUMS_FAST (include/geist_sampler_hip.h,
 * geist_hip_sampler_set_sums): whether the head's sampling calls form the sums of exponentials
 * with the reference's expf, bit for bit, or within the tolerance the sampling contract states.
 * No counterpart in the reference. */
int geist_hip_head_set_sums(struct geist_hip_head *h, int mode);
/* The same over the int8 form of the table, which the reference's x86 backend substitutes for
 * the F16 table in a decode step (src/backends/cpu_x86/backend.c:332-372): d_embed_q8 [vocab,
 * d_model] int8 and d_scales [vocab] as geist_hip_f16_to_q8w produces them, d_model a multiple
 * of 16. The logits equal those of the reference's q8w_gemv_m1 bit for bit. */
int geist_hip_head_project_finalize_q8w(struct geist_hip_head *h, const float *d_hidden,
                                        size_t ld_hidden, size_t k, const float *d_norm_weight,
                                        float rms_eps, const int8_t *d_embed_q8,
                                        const float *d_scales, size_t d_model,
                                        int32_t *out_tokens);
/* The same over a Q6_K table as it lies in a GGUF file (the tied embedding of the Gemma models,
 * whose logit soft-cap the head was created with): d_embed_q6k holds vocab rows of d_model / 256
 * super-blocks of 210 bytes, d_model a multiple of 256. The logits equal, bit for bit, those of
 * the reference's portable kernel cpu_scalar_w_quant_m1 / _mN after dequant_q6_K_row
 * (src/backends/cpu_scalar/weight_resolve.c:86-88, 186-241), for one row and for a batch. Unless
 * geist_hip_head_set_projection chose the portable backend,
 * one row gets the logits of the x86 backend's decode kernel q6k_gemv_m1 instead
 * (src/backends/cpu_x86/kernel_q6k_gemv.c, resolved at src/backends/cpu_x86/backend.c:395-397),
 * again bit for bit, and a batch those of its batch path cpu_x86_linear_q6k_mN
 * (src/backends/cpu_x86/linear_q6k.c:234-300; see geist_hip_q6k_packed_linear_x86_rows: as a host
 * with AVX-512 VNNI computes them, or in mode GEIST_HIP_PROJECTION_X86_AVX2 one without).
 * Q4_K: below. The
 * other formats the reference resolves for an embedding table (I2_S, an F32 table) have
 * no device kernel here: their callers project on the host or with their own kernel and pass
 * the logits to geist_hip_head_finalize_one_row / _batch.
 * geist_hip_head_reserve_projection_q6k is geist_hip_head_reserve_projection plus the scratch of
 * this kernel. geist_hip_head_q6k_load, once per model: keeps a copy of the table in the order
 * the device reads it (geist_hip_q6k_pack; 1 % more device memory than the table itself, the
 * x86 backend's counterpart being the int8 copy it builds at load) and reserves the buffers;
 * geist_hip_head_project_finalize_q6k with that same table pointer and d_model then streams the
 * copy (in the portable arithmetic 1.5 times as fast as the table, with the same logits bit for
 * bit). The packed copy is recognised by the table's address and d_model alone: the table is not
 * kept alive by the head, and after any change to its bytes -- a reload, merged adapter weights,
 * another table at the same address -- geist_hip_head_q6k_load must be called again, or the old
 * weights keep being used. */
int geist_hip_head_project_finalize_q6k(struct geist_hip_head *h, const float *d_hidden,
                                        size_t ld_hidden, size_t k, const float *d_norm_weight,
                                        float rms_eps, const void *d_embed_q6k, size_t d_model,
                                        int32_t *out_tokens);
int geist_hip_head_reserve_projection_q6k(struct geist_hip_head *h, size_t d_model);
int geist_hip_head_q6k_load(struct geist_hip_head *h, const void *d_embed_q6k, size_t d_model);
/* A Q4_K table (super-blocks of 144 bytes): geist_hip_head_q4k_load, once per model, keeps a
 * copy in the order the device reads it (geist_hip_q4k_pack, 3 % more device memory than the
 * table) and reserves the buffers; geist_hip_head_project_finalize_q4k with that same table
 * pointer and d_model then runs norm -> projection -> soft-cap -> sampler on the device.
 * Without the load the call is refused (GEIST_HIP_E_UNSUPPORTED): only the packed copy has a
 * kernel. The logits equal, bit for bit, those of the portable kernel cpu_scalar_w_quant_m1 /
 * _mN after dequant_q4_K_row (src/formats/gguf/q4_K.c:18-49, weight_resolve.c:82-83, 186-241),
 * for one row and for a batch. Unless geist_hip_head_set_projection chose the portable backend,
 * a vocabulary of a multiple of 8 tokens (d_model <= 16384) gets the logits of the x86 backend
 * instead (int8 activations, integer dot products): one row those of its decode kernel
 * q4kx8_gemv_m1 (src/backends/cpu_x86/kernel_q4kx8_gemm_avx512.c, from
 * src/backends/cpu_x86/linear_q4k.c:163-166), a batch those of cpu_x86_linear_q4k_mN
 * (linear_q4k.c:198-250; see geist_hip_q4k_packed_linear_x86_rows), again bit for bit. That
 * backend's W4A8 kernels for other shapes, and the NEON backend's kernels, are not reproduced. */
int geist_hip_head_project_finalize_q4k(struct geist_hip_head *h, const float *d_hidden,
                                        size_t ld_hidden, size_t k, const float *d_norm_weight,
                                        float rms_eps, const void *d_embed_q4k, size_t d_model,
                                        int32_t *out_tokens);
int geist_hip_head_q4k_load(struct geist_hip_head *h, const void *d_embed_q4k, size_t d_model);
/* The speculative output head of greedy decoding (src/archs/transformer/forward/spec_head.c;
 * include/geist_lm_head_hip.h has the device entry points). geist_hip_head_spec_build is
 * transformer_spec_head_init (spec_head.c:616-622) for a tied F16 table in device memory, which
 * must stay valid: it returns GEIST_HIP_E_UNSUPPORTED, and the head keeps no sketch, where the
 * reference or the device kernels build none. geist_hip_head_project_finalize_spec is
 * finalize_logits_one_row with the sketch in front (head.c:99-112) for one hidden row: output
 * norm, then the sketch head if the session is greedy and a sketch exists; when it declines
 * (verify != 0, as GEIST_SPEC_VERIFY=1, and an excluded row could have won) or does not apply,
 * the dense F16 head of geist_hip_head_project_finalize. *used_sketch (may be NULL) says which
 * of the two produced the token. */
int geist_hip_head_spec_build(struct geist_hip_head *h, const uint16_t *d_embed_f16, size_t d_model,
                              size_t stride_override, size_t topk_override);
int geist_hip_head_project_finalize_spec(struct geist_hip_head *h, const float *d_hidden,
                                         const float *d_norm_weight, float rms_eps,
                                         const uint16_t *d_embed_f16, size_t d_model, int verify,
                                         int32_t *out_token, int *used_sketch);
/* The logits of the last geist_hip_head_project_finalize[_q8w] call ([k, vocab], row stride vocab,
 * device memory; soft-cap not applied: the sampler applies it while reading), for scoring with
 * geist_hip_logprob_rows in place of geist_session_peek_logits. NULL before the first call and
 * after a token that the sketch head produced (there are no dense logits then: the reference
 * recomputes them on demand, arch.c:179; here the caller runs geist_hip_head_project_finalize). */
const float *geist_hip_head_logits(const struct geist_hip_head *h);

/* The drafting step of one speculative round (session.c:564-572) for a token history kept in
 * device memory: seed is the pending next token (what the finalize call of the step before
 * returned; op_peek_next_token, src/archs/transformer/arch.c:156-161), the drafts come from the
 * n-gram lookup with max_suffix = 4 (session.c:570-571). out_drafts holds k_max entries
 * (1..16); out_drafts[0] = seed. *match_len is the matched suffix length: the reference goes
 * on to verify_forward only when *n_drafts > 1 and *match_len >= 2 (session.c:572-592), and
 * falls back to a single decode step otherwise. */
int geist_hip_head_propose_drafts(struct geist_hip_head *h, const int32_t *d_history,
                                  size_t history_n, int32_t seed, size_t k_max,
                                  int32_t *out_drafts, size_t *n_drafts, size_t *match_len);

/* The accept step of one speculative round. drafts[0..k) are the tokens fed to verify_forward
 * (drafts[0] is the already-sampled next token, session.c:563-568), d_logits the [k, vocab] rows
 * it produced: row i holds the logits for the position after drafts[i].
 *   GEIST_HIP_SPEC_REFERENCE  the reference's loop: every row is sampled with the session's
 *       sampler (one shared RNG, row order, as finalize_logits_batch), the longest prefix with
 *       sampled[i] == drafts[i + 1] is accepted and sampled[accepted] is the correction
 *       (session.c:599-625). Under T > 0 the stream is valid but not distribution-preserving
 *       (include/geist_util.h:233-240).
 *   GEIST_HIP_SPEC_REJECTION  T > 0 with no top-k / top-p filter: rejection sampling against the
 *       n-gram drafter's point-mass proposals -- draft i+1 is accepted with probability
 *       p_i(drafts[i+1]); at the first rejection the correction is drawn from p_i with that
 *       token struck out; if all are accepted the bonus is a temperature draw from row k-1. The
 *       emitted stream then has the distribution of k decode_step calls. Consumes k draws of
 *       the session's RNG, like the reference mode. T == 0 behaves as the reference mode;
 *       a filter set with T > 0 returns GEIST_E_UNSUPPORTED (7).
 * Writes drafts[0..accepted], then the correction: n_out = accepted + 2 tokens in all,
 * out_capacity >= k + 1 (include/geist_util.h:226). The caller truncates its KV cache to the
 * accepted prefix and prefills the correction as the reference does (session.c:611-632). */
#define GEIST_HIP_SPEC_REFERENCE 0
#define GEIST_HIP_SPEC_REJECTION 1
int geist_hip_head_spec_accept(struct geist_hip_head *h, const float *d_logits, size_t k,
                               const int32_t *drafts, int mode, size_t out_capacity,
                               int32_t *out_tokens, size_t *n_out);

/* Current RNG state (for tests and for handing a session over). */
int geist_hip_head_rng_state(struct geist_hip_head *h, uint64_t *state);

#ifdef __cplusplus
}
#endif
#endif /* GEIST_HEAD_HIP_H */
