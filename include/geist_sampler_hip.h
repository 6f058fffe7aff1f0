/*
 * geist_sampler_hip.h -- C ABI of the MI355X (gfx950) token-sampling path.
 *
 * Plain C: pointers and sizes only. Logit rows [rows x n_vocab] fp32 stay resident in device
 * memory; every entry point enqueues hand-written HIP kernels on the sampler's stream and
 * returns (asynchronous unless stated otherwise). There is no CPU fallback: when no device
 * or no kernel image for it is available the calls fail with GEIST_E_BACKEND.
 *
 * Each declaration cites the interface of the reference (geistlib 0.9.0, paths relative to
 * its tree) that it replaces or extends.
 */
#ifndef GEIST_SAMPLER_HIP_H
#define GEIST_SAMPLER_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes: numerically identical to `enum geist_status` (include/geist.h:46-67), so a
 * caller compiled against the reference header can return them unchanged. */
#define GEIST_HIP_OK 0
#define GEIST_HIP_E_OOM 1
#define GEIST_HIP_E_INVALID_ARG 2
#define GEIST_HIP_E_INTERNAL 3
#define GEIST_HIP_E_UNSUPPORTED 7
#define GEIST_HIP_E_BACKEND 9

/* geist_token_t (include/geist.h:190) */
typedef int32_t geist_hip_token_t;

typedef struct geist_hip_sampler geist_hip_sampler;

/* Replaces geist_sampler_workspace_init (src/engine/sampler.h:50-57, sampler.c:136-148): the
 * caller-owned scratch of the reference becomes a device workspace sized once for
 * `max_rows` rows of up to `max_vocab` logits. `stream` is a hipStream_t (NULL = the
 * device's default stream). All later calls on this object run on that stream; one object
 * per host thread, as one workspace per session in the reference. */
int geist_hip_sampler_create(int device, size_t max_rows, size_t max_vocab, void *stream,
                             geist_hip_sampler **out);
/* Replaces geist_sampler_workspace_destroy (sampler.c:150-157). NULL is a no-op. */
void geist_hip_sampler_destroy(geist_hip_sampler *s);
/* Text of the last failure on this object (the reference keeps such text in per-handle
 * error slots, src/base/error.h:34-39). Never NULL. */
const char *geist_hip_sampler_last_error(const geist_hip_sampler *s);
/* Blocks until everything enqueued on the sampler's stream has finished. */
int geist_hip_sampler_sync(geist_hip_sampler *s);

/* The reference's sample call returns with the token (forward/head.c:165-186). Here the ids of a
 * sampling call are written by kernels, and a caller that waits for the stream pays the runtime's
 * completion path on top of them. With enable = 1 every sampling call of `s` also stores, after
 * the ids of all its rows, the call's number into a word of page-locked host memory -- the kernel
 * that writes the last id does it where the step is one launch, a launch of its own otherwise.
 * geist_hip_sampler_wait_ids() then watches that word: it returns as soon as the ids of the last
 * call enqueued are written (meant for ids that go to page-locked memory, geist_hip_host_malloc,
 * which the host can then read at once) and falls back to waiting for the stream -- which also
 * reports a failed launch -- when the word has not changed within a bounded time
 * (geist_hip_sampler_set_wait_spin, default 2000 us; 0 = do not watch at all). With enable = 0
 * (the default) wait_ids is geist_hip_sampler_sync. Other work enqueued on the stream after the
 * sampling call is not waited for. */
int geist_hip_sampler_notify_ids(geist_hip_sampler *s, int enable);
int geist_hip_sampler_wait_ids(geist_hip_sampler *s);
int geist_hip_sampler_set_wait_spin(geist_hip_sampler *s, uint32_t microseconds);
/* Rebinds the stream later calls are enqueued on (NULL = default stream). */
int geist_hip_sampler_set_stream(geist_hip_sampler *s, void *stream);

/* Where the logits of the following calls are expected to be when they are read (no reference
 * counterpart: the reference samples from host memory).
 *   GEIST_HIP_LOGITS_CACHED    (default) they were written just before, by an lm_head on the same
 *                              device, and may still be in the Infinity Cache: ordinary loads.
 *   GEIST_HIP_LOGITS_STREAMED  they come from HBM (a batch larger than the cache, rows gathered
 *                              from several producers, a buffer that has been idle): the single
 *                              pass of the greedy and top-k modes reads them with non-temporal
 *                              loads, ~8 % faster from HBM and ~60 % slower if the rows were
 *                              cached after all. Results are identical either way. */
#define GEIST_HIP_LOGITS_CACHED 0
#define GEIST_HIP_LOGITS_STREAMED 1
int geist_hip_sampler_set_logits_hint(geist_hip_sampler *s, int hint);

/* A batch of logit rows in device memory. Row r starts at d_logits + r * ld.
 * The optional token history drives the penalties: row r owns d_history[r * history_ld ..
 * + d_history_len[r]) ; ids outside [0, n_vocab) are ignored.
 * The optional allowed-token mask is the device form of constrained decoding, which the
 * reference leaves to a runtime that reads the logits back, masks what its grammar forbids and
 * samples itself (docs/API_CONTRACT.md:35-44; geist_session_peek_logits,
 * include/geist_util.h:195-211): bit (e % 32) of word d_allowed[r * allowed_ld + e / 32] set =
 * token e may be sampled in row r; a forbidden token's logit is -inf, after the penalties and
 * the soft-cap (peek_logits hands out capped values), in every mode, greedy included.
 * allowed_ld = 0: one mask of (n_vocab + 31) / 32 words shared by all rows. Every row must
 * allow at least one token with a logit above -inf. */
struct geist_hip_rows {
    const float    *d_logits;
    size_t          ld;
    size_t          rows;
    size_t          n_vocab;
    const int32_t  *d_history;     /* NULL = no history */
    size_t          history_ld;
    const int32_t  *d_history_len; /* rows entries */
    const uint32_t *d_allowed;     /* NULL = every token allowed */
    size_t          allowed_ld;    /* words between the masks of consecutive rows; 0 = shared */
};

/* Sampling configuration for one call. The first four fields are the sampler fields of
 * `struct geist_session_opts` (include/geist.h:213-229) after
 * transformer_session_apply_opts (src/archs/transformer/forward/step.c:385-411).
 *
 * precedence:
 *   GEIST_HIP_PRECEDENCE_REFERENCE  the reference's dispatch (head.c:172-183): T == 0 -> argmax;
 *                                   top_k > 1 -> top-k (top_p ignored); 0 < top_p < 1 -> top-p;
 *                                   else temperature. min_p must be 0.
 *   GEIST_HIP_PRECEDENCE_CHAIN      temperature -> top-k -> top-p -> min-p composed, each filter
 *                                   acting on the survivors of the previous one. With a single
 *                                   filter set it gives the same token as the reference mode.
 * Penalties (history present and any of the three non-neutral) and the soft-cap
 * (tanhf(x / cap) * cap, head.c:148-159; applied only when T > 0) act on the logits before
 * either precedence, without writing to d_logits. */
#define GEIST_HIP_PRECEDENCE_REFERENCE 0
#define GEIST_HIP_PRECEDENCE_CHAIN 1
struct geist_hip_sample_params {
    float temperature;
    float top_p;
    int   top_k;
    float min_p;
    float repetition_penalty; /* 1 = neutral */
    float frequency_penalty;  /* 0 = neutral */
    float presence_penalty;   /* 0 = neutral */
    float logit_softcap;      /* 0 = off */
    int   precedence;
};

/* Replaces the sampler dispatch of finalize_logits_batch (head.c:274-304) for `rows` rows at
 * once: d_out_tokens[r] = token sampled from row r with the uniform d_uniforms[r] (the value
 * geist_rng_next_unit would have returned for that row). d_uniforms may be NULL when the
 * configuration is greedy. */
int geist_hip_sample_rows(geist_hip_sampler *s, const struct geist_hip_rows *rows,
                          const struct geist_hip_sample_params *params, const float *d_uniforms,
                          geist_hip_token_t *d_out_tokens);

/* geist_hip_sample_rows for callers that cannot allocate. It has no counterpart in the reference;
 * it is for code under HIP graph capture, tight serving loops and harnesses that forbid
 * hipMalloc: no sampler object is needed and the call allocates nothing, on the host or on the
 * device. Its workspace is an array of device memory inside the library's code object
 * (7.3 MiB per GPU, held until the process ends).
 *   device, stream   where the kernels are enqueued (stream NULL = the default stream)
 *   err, err_len     optional buffer for the text of a failure
 * Served: greedy, temperature, and every top-k configuration (with top-p / min-p behind it,
 * penalties, soft-cap, allowed-token mask). Top-p / min-p WITHOUT top-k returns
 * GEIST_HIP_E_UNSUPPORTED. rows x ceil(n_vocab / 2048) must not exceed
 * GEIST_HIP_STATIC_MAX_UNITS (e.g. 64 rows of 128256 logits), else GEIST_HIP_E_INVALID_ARG.
 * Same tokens as geist_hip_sample_rows. All calls on one GPU share the one array: calls that
 * overlap on a GPU (two streams, two threads) race; calls on one stream are ordered. The first
 * call on a device looks the array's address up (geist_hip_sampler_create does so too). */
#define GEIST_HIP_STATIC_MAX_UNITS 4096
int geist_hip_sample_rows_static(int device, void *stream, const struct geist_hip_rows *rows,
                                 const struct geist_hip_sample_params *params,
                                 const float *d_uniforms, geist_hip_token_t *d_out_tokens,
                                 char *err, size_t err_len);

/* No counterpart in the reference. The modes that need a row's maximum before they can sum its
 * exponentials (temperature, top-p, min-p, softmax, speculative verification) read the rows
 * once: the workgroups that share a row wait for one another inside the kernel. `polls` bounds
 * that wait (default 65536 polls, tens of milliseconds); a workgroup that reaches the bound
 * finds the row's maximum by reading the row itself, so the results never depend on it. 0 makes
 * every workgroup do that at once, which is slow and meant for tests of that path. */
int geist_hip_sampler_set_wait_limit(geist_hip_sampler *s, uint32_t polls);

/* No counterpart in the reference. The top-k candidate path runs as one launch (the workgroup of
 * a row that finishes scanning last goes on as the row's final stage) when the batch
 * fits the device in one round of workgroups and the device places the
 * workgroups of a row where they share a second-level cache (looked at once per device: it
 * decides which form is faster, not whether the one launch is correct -- every launch checks the
 * placement of each row for itself, see geist_hip_sampler_handoff_scope); otherwise as two
 * launches. Results are the same either way. enable = 0 keeps to two launches, 1 returns to the
 * default. Returns 1 when the one-launch form is in use for batches that qualify, 0 when not,
 * negative on error. */
int geist_hip_sampler_one_launch_topk(geist_hip_sampler *s, int enable);

/* No counterpart in the reference. A top-p / min-p row whose kept prefix is too long for the
 * candidate list (tens of thousands of entries: a flat row at a high temperature) is walked in
 * full, as sampler.c:246-304 sorts and walks it. One workgroup takes 275 to 300 us for a row of
 * 128 k logits; spread over the workgroups of the row's chunks, which keep their part of the row
 * in registers and meet after every pass, the walk takes a fifth of that -- at the price of one
 * more launch per call.
 *   GEIST_HIP_WHOLE_ROW_WALK_ADAPTIVE       (default) the extra launch is sent while such rows
 *                                           keep turning up: the kernels report them in a
 *                                           page-locked word that the next call looks at
 *   GEIST_HIP_WHOLE_ROW_WALK_SPREAD         always send it
 *   GEIST_HIP_WHOLE_ROW_WALK_ONE_WORKGROUP  never
 * Tokens are the same in every mode. geist_hip_sampler_row_paths reports 3 for a row walked by
 * one workgroup, 4 for a row walked by its chunks' workgroups. The waits of the spread form are
 * bounded by geist_hip_sampler_set_wait_limit like those of the one-pass kernels: a row whose
 * workgroups do not all turn up in time is walked by its first workgroup alone. */
#define GEIST_HIP_WHOLE_ROW_WALK_ADAPTIVE 0
#define GEIST_HIP_WHOLE_ROW_WALK_SPREAD 1
#define GEIST_HIP_WHOLE_ROW_WALK_ONE_WORKGROUP 2
int geist_hip_sampler_set_whole_row_walk(geist_hip_sampler *s, int mode);

/* No counterpart in the reference. In the one-launch form the workgroups of a row hand their
 * candidates to the one that finishes the row, through plain stores that are only sure to be
 * seen inside the second-level cache of the XCD that wrote them. Each arrival reports the XCD it
 * ran on; when all of a row ran on one XCD the finishing workgroup reads the hand-over from the
 * cache they share, otherwise it leaves the hand-over unread and finds the row's candidates from
 * the logits themselves. always_agent = 1 makes every row take the second branch whatever its
 * placement -- for tests of that branch; 0 returns to the default. Results are the same either
 * way.
 * The one-pass kernels (temperature, top-p / min-p, verification) use the same cache for the
 * slots through which the workgroups of a row meet, where the launch deals a row to one XCD
 * (a row count that is a multiple of 8, and the one-kernel temperature draw): plain stores, which
 * that XCD's cache serves to the polling workgroups. Workgroups that did not share an XCD would
 * not see one another, their bounded waits would run out and each would read the row itself:
 * slower, the same ids. always_agent = 1 makes these stores device-scope as well. */
int geist_hip_sampler_handoff_scope(geist_hip_sampler *s, int always_agent);

/* No counterpart in the reference. The modes that weigh every element (temperature, top-p /
 * min-p over the whole vocabulary, normalised probabilities, speculative verification) form a
 * row's sum of exponentials with the reference's own expf, bit for bit, so that every id is the
 * reference's (GEIST_HIP_SUMS_EXACT, the default). GEIST_HIP_SUMS_FAST forms the SUMS from the
 * hardware's 2^z instead (relative error of a sum about 1e-7); every weight that is compared
 * with a share of a sum -- in the walks, the nucleus, the acceptance test -- stays exact. An id
 * can then differ from the reference's only where the reference's own decision lies within that
 * error of an edge (a draw within 1e-7 of a slot's edge, a nucleus that ends within 1e-7 of
 * top_p): the tolerance the sampling contract states, used. The pass over the logits gets a
 * fifth to a third shorter (without penalties and without a min-p list the workgroups of a row
 * then do not wait for one another either: each sums against its chunk's maximum and a small
 * launch scales the sums to the row's). Which rows those are is not reported: a caller that has to know compares with
 * the exact mode. The one-kernel temperature draw of a few rows and the top-k path form no such
 * sums and are exact in both modes. */
#define GEIST_HIP_SUMS_EXACT 0
#define GEIST_HIP_SUMS_FAST 1
int geist_hip_sampler_set_sums(geist_hip_sampler *s, int mode);

/* No counterpart in the reference. Stochastic speculative verification sums the residual
 * max(0, p - q) and draws from it in one launch (the workgroups of a sequence wait for one
 * another's sums, the wait bounded by geist_hip_sampler_set_wait_limit) when sequences x chunks
 * of 8192 logits is at most two per compute unit (512 on an MI355X), one round of that kernel's
 * workgroups; otherwise, and with enable = 0, in two launches. Results are the same either way. Returns 1 when the one-launch
 * form is in use for batches that qualify, 0 when not, negative on error. */
int geist_hip_sampler_one_launch_spec(geist_hip_sampler *s, int enable);

/* Sizes, ahead of the first sampling call, whatever workspace the configuration needs beyond
 * what geist_hip_sampler_create made -- the reference sizes its workspace when the options are
 * applied (transformer_session_apply_opts, src/archs/transformer/forward/step.c:398-409), so that
 * the per-token call allocates nothing. Today that is the full-vocabulary top-p / min-p path (a
 * row of probabilities per logit row). n_vocab = 0: the sampler's max_vocab. A sampling call
 * made without it sizes the same workspace on first use. */
int geist_hip_sampler_prepare(geist_hip_sampler *s, const struct geist_hip_sample_params *params,
                              size_t n_vocab);

/* Same, drawing the uniforms on the device from xorshift64* states (struct geist_rng,
 * src/engine/sampler.h:28-32; sampler.c:35-48) held in device memory.
 *   shared != 0: one state for the whole batch, row r takes the (r+1)-th draw and the state
 *                advances by `rows` draws -- the reference's batch order (head.c:274-304).
 *   shared == 0: d_rng_states[r] belongs to row r and advances by one draw.
 * Greedy configurations leave the states untouched (sampler.c:110-112, 184-186, 238-240). */
int geist_hip_sample_rows_rng(geist_hip_sampler *s, const struct geist_hip_rows *rows,
                              const struct geist_hip_sample_params *params,
                              uint64_t *d_rng_states, int shared,
                              geist_hip_token_t *d_out_tokens);

/* Fills the backend slot `argmax_f32` (include/geist_backend.h:414-421): greedy argmax over one
 * fp32 row of n logits in device memory, lowest index wins ties; synchronous, only the 4-byte
 * index crosses to the host. */
int geist_hip_argmax_f32(geist_hip_sampler *s, const float *d_logits, size_t n,
                         int32_t *out_index);

/* Penalties applied IN PLACE to the rows (the caller-side mutation the reference performs for
 * its soft-cap, head.c:148-159). For each distinct history id t of a row with count c:
 *   l = logits[t]; l = l > 0 ? l / rep : l * rep; l -= freq * c; l -= pres.
 * No reference counterpart (the reference has no penalties). */
int geist_hip_apply_penalties(geist_hip_sampler *s, float *d_logits, size_t ld, size_t rows,
                              size_t n_vocab, const int32_t *d_history, size_t history_ld,
                              const int32_t *d_history_len, float rep, float freq, float pres);

/* Normalised probabilities of each row after penalties, soft-cap and temperature, the values
 * the reference's top-p path holds in ws->probs after sampler.c:246-253:
 *   d_probs[r * ld_probs + i] = (float)((double)expf((l_i - max) / T) / sum). */
int geist_hip_softmax_rows(geist_hip_sampler *s, const struct geist_hip_rows *rows,
                           const struct geist_hip_sample_params *params, float *d_probs,
                           size_t ld_probs);

/* Scoring without moving logits to the host. Replaces geist_session_peek_logits
 * (include/geist_util.h:195-211; src/archs/transformer/arch.c:167-197, which hands out the
 * soft-capped values) followed by the log-softmax lookup of the reference's evaluation tool
 * (logprob_at, tools/eval_geist.c:63-73), for k_per_row candidate tokens of each row:
 *   d_out[r * out_ld + j] = (double)(l[t] - max) - log(sum_i exp((double)(l_i - max))),
 *   t = d_tokens[r * tokens_ld + j], l = the row after tanhf(x / cap) * cap when cap > 0.
 * Token ids outside [0, n_vocab) give NaN. No penalties, no temperature: peek_logits exposes the
 * model's values. Double results; against the CPU statement they differ only by the order of the
 * double sum and the last bit of exp/log (bound 1e-9 absolute in the tests). */
int geist_hip_logprob_rows(geist_hip_sampler *s, const float *d_logits, size_t ld, size_t rows,
                           size_t n_vocab, float logit_softcap, const int32_t *d_tokens,
                           size_t tokens_ld, size_t k_per_row, double *d_out, size_t out_ld);

/* The n-gram drafter of the reference's speculative loop (propose_drafts_ngram,
 * src/engine/session.c:437-513; called with max_suffix = 4 at :570-571, capped at 8 at :455-456), for n_seq sequences
 * whose token histories are on the device (the history layout of struct geist_hip_rows):
 *   d_history [n_seq][history_ld], d_history_len [n_seq], d_seed [n_seq] (each sequence's
 *   pending next token, op_peek_next_token, src/archs/transformer/arch.c:156-161: here the
 *   output of the geist_hip_sample_rows call of the step before, still on the device)
 * Finds the longest suffix of history + [seed], at most min(max_suffix, 8) tokens, that occurs
 * earlier in the history; among the occurrences of that length the one with the most following
 * tokens (counted up to k_max - 1), the most recent among equals.
 *   d_out_drafts [n_seq][out_ld]: drafts[0] = seed, then the tokens that followed the match
 *   d_out_count  [n_seq]: number of drafts written (>= 1; 1 = no usable match)
 *   d_out_match_len [n_seq]: length of the matched suffix, 0 without a match (the reference
 *                    skips verification below GEIST_SPEC_MIN_L = 2, session.c:575-592)
 * 1 <= k_max <= 16 (GEIST_SPEC_KMAX_HARDCAP, session.c:515), out_ld >= k_max. */
int geist_hip_propose_drafts_ngram(geist_hip_sampler *s, const int32_t *d_history,
                                   size_t history_ld, const int32_t *d_history_len,
                                   const geist_hip_token_t *d_seed, size_t n_seq, size_t k_max,
                                   size_t max_suffix, geist_hip_token_t *d_out_drafts,
                                   size_t out_ld, int32_t *d_out_count, int32_t *d_out_match_len);

/* Speculative-decode verification for n_seq sequences with draft length L (no reference
 * counterpart: include/geist_util.h:233-240 documents that the reference's speculative loop
 * omits rejection sampling; the batch shape is that of verify_forward,
 * src/archs/transformer/arch_ops.c:176-270).
 *   d_target   [n_seq][L+1][n_vocab] logits, sequence stride (L+1)*ld_t, row stride ld_t
 *   d_draft_q  [n_seq][L][n_vocab] draft probabilities, row stride ld_q; NULL when the drafter
 *              proposes with certainty (the reference's n-gram lookup, session.c:437-513):
 *              q_j is then 1 at the draft token, a draft is accepted with probability p_j(x_j)
 *              and the resample is p_j with x_j struck out
 *   d_draft    [n_seq][L] draft token ids,  d_uniforms [n_seq][L+1]
 * T > 0: position j accepted iff u_j * q_j(x_j) < p_j(x_j); at the first rejection the token is
 * drawn with u_L from max(0, p_j - q_j) renormalised; if all are accepted the bonus token is a
 * temperature draw from row L with u_L. T <= 0: exact-match against the row argmax.
 * logit_softcap > 0: the target rows are capped (tanhf(x / cap) * cap, head.c:148-159) before
 * anything else when T > 0, as the reference caps them before it samples.
 *   d_out_tokens [n_seq][L+1]: accepted draft ids, then the emitted token; rest untouched.
 *   d_n_accepted [n_seq]. */
int geist_hip_spec_verify(geist_hip_sampler *s, const float *d_target, size_t ld_t,
                          const float *d_draft_q, size_t ld_q, const int32_t *d_draft,
                          const float *d_uniforms, size_t n_seq, size_t L, size_t n_vocab,
                          float temperature, float logit_softcap,
                          geist_hip_token_t *d_out_tokens, int32_t *d_n_accepted);

/* n consecutive geist_rng_next_unit values (sampler.c:44-48) from the state at d_rng_state (a
 * struct geist_rng in device memory), written to d_out_units; the state advances by n draws. */
int geist_hip_rng_draw_units(geist_hip_sampler *s, uint64_t *d_rng_state, size_t n,
                             float *d_out_units);

/* ---- small device-memory helpers so that a plain-C host needs no HIP headers -------------- */
int geist_hip_malloc(geist_hip_sampler *s, size_t bytes, void **d_ptr);
int geist_hip_free(geist_hip_sampler *s, void *d_ptr);
int geist_hip_upload(geist_hip_sampler *s, void *d_dst, const void *h_src, size_t bytes);   /* sync */
int geist_hip_download(geist_hip_sampler *s, void *h_dst, const void *d_src, size_t bytes); /* sync */
/* Page-locked host memory that the device reads and writes in place (the same pointer on both
 * sides): a kernel's stores are in host memory once the stream has been waited for
 * (geist_hip_sampler_sync), the host's stores are read by kernels launched afterwards. For the
 * few words of results and arguments of a decode step, which then need no copy command. */
int geist_hip_host_malloc(geist_hip_sampler *s, size_t bytes, void **h_ptr);
int geist_hip_host_free(geist_hip_sampler *s, void *h_ptr);

/* Diagnostics (no reference counterpart): after a full-vocabulary top-p / min-p call, which walk
 * served each row: 1 = shortcut over the per-thread maxima, 2 = candidate list, 3 = the whole
 * row. Synchronous; h_paths receives `rows` entries. */
int geist_hip_sampler_row_paths(geist_hip_sampler *s, int32_t *h_paths, size_t rows);

/* Diagnostics (no reference counterpart): after a top-k call, which path served each row:
 * 0 = the candidates handed on by the scan, 1 = the per-thread maxima (rows whose leading logits
 * crowd into few wavefronts' elements, runs of equal values), 2 = the selection over the whole
 * row; -1 for every row when the call did not take the candidate path at all (soft-cap, mask,
 * unaligned rows, k above 64, penalties that can raise a logit). Synchronous. */
int geist_hip_sampler_topk_paths(geist_hip_sampler *s, int32_t *h_paths, size_t rows);

#ifdef __cplusplus
}
#endif
#endif /* GEIST_SAMPLER_HIP_H */
