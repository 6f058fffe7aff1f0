/*
 * bench_hooks.hip -- timing helpers for bench.py (see geist_bench_hip.h). Links against the
 * product library for the staged sampling call; the calibration kernel lives here.
 */
#include "geist_bench_hip.h"

#include <hip/hip_runtime.h>

#include <cstdio>
#include <time.h>
#include <cstring>
#include <new>

#include "../csrc/sampler_device.h"
#include "../csrc/sampler_host.h"

struct geist_bench_timer {
    hipEvent_t  a, b;
    hipStream_t stream;
};

namespace {

/* reads a row's chunk [8192 * chunk, +8192) as the streaming kernels do; nothing is written (a
 * maximum nobody stores keeps the loads alive) */
__global__ __launch_bounds__(gs::TPB) void k_plain_read(gs::RowView rv, float *__restrict__ sink) {
    int row = blockIdx.y, chunk = blockIdx.x;
    if ((gridDim.y & 7) == 0) { /* the rows dealt out over the XCDs as the sampling kernels do */
        const int lin = blockIdx.y * gridDim.x + blockIdx.x, slot = lin >> 3;
        row           = (lin & 7) + 8 * (slot / (int) gridDim.x);
        chunk         = slot % (int) gridDim.x;
    }
    const int base = chunk * rv.per_chunk;
    const int end  = base + rv.per_chunk < rv.n_vocab ? base + rv.per_chunk : rv.n_vocab;
    float4    v[8];
    gs::load_raw<8>(rv, rv.logits + (long) row * rv.ld, base, end, v);
    float m = -__builtin_inff();
#pragma unroll
    for (int j = 0; j < 8; ++j)
        m = gs::max3f(m, gs::max3f(v[j].x, v[j].y, v[j].z), v[j].w);
    if (m == 0x1.234568p+100f) /* never among the inputs */
        sink[0] = m;
}

float *g_sink = nullptr;

} // namespace

extern "C" {

int geist_bench_timer_begin(void *stream, geist_bench_timer **out) {
    if (!out)
        return GEIST_HIP_E_INVALID_ARG;
    geist_bench_timer *t = new (std::nothrow) geist_bench_timer;
    if (!t)
        return GEIST_HIP_E_OOM;
    t->stream = (hipStream_t) stream;
    if (hipEventCreate(&t->a) != hipSuccess) {
        delete t;
        return GEIST_HIP_E_BACKEND;
    }
    if (hipEventCreate(&t->b) != hipSuccess) {
        (void) hipEventDestroy(t->a);
        delete t;
        return GEIST_HIP_E_BACKEND;
    }
    if (hipEventRecord(t->a, t->stream) != hipSuccess) {
        (void) hipEventDestroy(t->a);
        (void) hipEventDestroy(t->b);
        delete t;
        return GEIST_HIP_E_BACKEND;
    }
    *out = t;
    return GEIST_HIP_OK;
}

int geist_bench_timer_end(geist_bench_timer *t, double *ms) {
    if (!t)
        return GEIST_HIP_E_INVALID_ARG;
    float f  = 0.0f;
    int   rc = GEIST_HIP_OK;
    if (hipEventRecord(t->b, t->stream) != hipSuccess || hipEventSynchronize(t->b) != hipSuccess ||
        hipEventElapsedTime(&f, t->a, t->b) != hipSuccess)
        rc = GEIST_HIP_E_BACKEND;
    (void) hipEventDestroy(t->a);
    (void) hipEventDestroy(t->b);
    delete t;
    if (ms)
        *ms = f;
    return rc;
}

int geist_bench_time_stream_kernel(geist_hip_sampler *s, void *stream,
                                   const struct geist_hip_rows *rows, size_t n_batches,
                                   const struct geist_hip_sample_params *params,
                                   const float *d_uniforms, geist_hip_token_t *d_out_tokens,
                                   int launches, double *ms_total, char *kernel_name,
                                   size_t kernel_name_len) {
    if (!s || !rows || n_batches < 1 || launches < 1 || !ms_total)
        return GEIST_HIP_E_INVALID_ARG;
    const char *name = "";
    int         rc   = 0;
    for (size_t i = 0; i < n_batches && !rc; ++i)
        rc = gs_host::sample_stages(s, &rows[i], params, d_uniforms, d_out_tokens,
                                    gs_host::STAGE_ALL, nullptr);
    for (size_t i = 0; i < n_batches && !rc; ++i) /* warms the code object, cycles the caches */
        rc = gs_host::sample_stages(s, &rows[i], params, d_uniforms, d_out_tokens,
                                    gs_host::STAGE_STREAM, &name);
    if (rc)
        return rc;
    geist_bench_timer *t = nullptr;
    rc                   = geist_bench_timer_begin(stream, &t);
    for (int i = 0; i < launches && !rc; ++i)
        rc = gs_host::sample_stages(s, &rows[(size_t) i % n_batches], params, d_uniforms,
                                    d_out_tokens, gs_host::STAGE_STREAM, nullptr);
    if (t) {
        const int rc2 = geist_bench_timer_end(t, ms_total);
        rc            = rc ? rc : rc2;
    }
    if (kernel_name && kernel_name_len)
        snprintf(kernel_name, kernel_name_len, "%s", name);
    return rc;
}

int geist_bench_step_latency(geist_hip_sampler *s, const struct geist_hip_rows *rows,
                             size_t n_batches, const struct geist_hip_sample_params *params,
                             const float *d_uniforms, geist_hip_token_t *out_tokens, int wait_ids,
                             int samples, double *us_each) {
    if (!s || !rows || n_batches < 1 || samples < 1 || !us_each)
        return GEIST_HIP_E_INVALID_ARG;
    for (int i = 0; i < samples; ++i) {
        struct timespec t0, t1;
        clock_gettime(CLOCK_MONOTONIC, &t0);
        int rc = geist_hip_sample_rows(s, &rows[(size_t) i % n_batches], params, d_uniforms,
                                       out_tokens);
        if (rc == GEIST_HIP_OK)
            rc = wait_ids ? geist_hip_sampler_wait_ids(s) : geist_hip_sampler_sync(s);
        clock_gettime(CLOCK_MONOTONIC, &t1);
        if (rc != GEIST_HIP_OK)
            return rc;
        us_each[i] = (double) (t1.tv_sec - t0.tv_sec) * 1e6 + (double) (t1.tv_nsec - t0.tv_nsec) * 1e-3;
    }
    return GEIST_HIP_OK;
}

int geist_bench_time_plain_read(void *stream, const struct geist_hip_rows *rows, size_t n_batches,
                                int streamed, int launches, double *ms_total) {
    if (!rows || n_batches < 1 || launches < 1 || !ms_total)
        return GEIST_HIP_E_INVALID_ARG;
    if (!g_sink && hipMalloc((void **) &g_sink, 64) != hipSuccess)
        return GEIST_HIP_E_OOM;
    auto launch = [&](const struct geist_hip_rows &r) {
        gs::RowView rv = {};
        rv.logits      = r.d_logits;
        rv.ld          = (long) r.ld;
        rv.n_vocab     = (int) r.n_vocab;
        rv.per_chunk   = 8192;
        rv.n_chunks    = (int) ((r.n_vocab + 8191) / 8192);
        rv.vec_ok      = (((uintptr_t) r.d_logits) % 16 == 0) && (r.ld % 4 == 0);
        rv.stream_loads = streamed;
        k_plain_read<<<dim3(rv.n_chunks, (unsigned) r.rows), dim3(gs::TPB), 0, (hipStream_t) stream>>>(
            rv, g_sink);
    };
    for (size_t i = 0; i < n_batches; ++i)
        launch(rows[i]);
    geist_bench_timer *t = nullptr;
    int                rc = geist_bench_timer_begin(stream, &t);
    for (int i = 0; i < launches && !rc; ++i)
        launch(rows[(size_t) i % n_batches]);
    if (t) {
        const int rc2 = geist_bench_timer_end(t, ms_total);
        rc            = rc ? rc : rc2;
    }
    if (!rc && hipGetLastError() != hipSuccess)
        rc = GEIST_HIP_E_BACKEND;
    return rc;
}

} /* extern "C" */
