/*
 * geist_bench_hip.h -- timing helpers for bench.py, built into libgeist_bench_hip.so. They are
 * not part of the product's C ABI (include/) and nothing in the product libraries calls them.
 * All durations come from HIP events recorded on the stream the timed work is enqueued on.
 */
#ifndef GEIST_BENCH_HIP_H
#define GEIST_BENCH_HIP_H

#include "../../include/geist_sampler_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* A timed region on `stream` (a hipStream_t, NULL = the default stream): begin records the first
 * event, end records the second, waits for it and returns the milliseconds between them. */
typedef struct geist_bench_timer geist_bench_timer;
int geist_bench_timer_begin(void *stream, geist_bench_timer **out);
int geist_bench_timer_end(geist_bench_timer *t, double *ms);

/* Mean-duration measurement of the logit-streaming kernel of a configuration on its own:
 * enqueues only that kernel `launches` times back to back on `stream` (the stream `s` was made
 * with), launch i reading rows[i % n_batches], and returns the total milliseconds. One complete
 * sampling call per batch is made first (so that the kernel finds what an earlier pass leaves it),
 * then one untimed round of the kernel alone. kernel_name receives the kernel's name. */
int geist_bench_time_stream_kernel(geist_hip_sampler *s, void *stream,
                                   const struct geist_hip_rows *rows, size_t n_batches,
                                   const struct geist_hip_sample_params *params,
                                   const float *d_uniforms, geist_hip_token_t *d_out_tokens,
                                   int launches, double *ms_total, char *kernel_name,
                                   size_t kernel_name_len);

/* One-step latency measured from C: `samples` times geist_hip_sample_rows on rows[i % n_batches]
 * followed by geist_hip_sampler_wait_ids (wait_ids != 0) or geist_hip_sampler_sync, each timed
 * with clock_gettime(CLOCK_MONOTONIC) from before the call to after the wait; us_each receives
 * the microseconds of every sample. */
int geist_bench_step_latency(geist_hip_sampler *s, const struct geist_hip_rows *rows,
                             size_t n_batches, const struct geist_hip_sample_params *params,
                             const float *d_uniforms, geist_hip_token_t *out_tokens, int wait_ids,
                             int samples, double *us_each);

/* Calibration: the same loop around a kernel that only reads the rows (8192 logits per workgroup
 * of 256 threads, 16-byte loads, non-temporal when `streamed`) and stores nothing: the floor of
 * any one-pass kernel over these bytes on this device. */
int geist_bench_time_plain_read(void *stream, const struct geist_hip_rows *rows, size_t n_batches,
                                int streamed, int launches, double *ms_total);

#ifdef __cplusplus
}
#endif
#endif
