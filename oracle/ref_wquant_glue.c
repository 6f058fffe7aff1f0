/*
 * ref_wquant_glue.c -- TEST INFRASTRUCTURE: calls the reference's portable linear kernels
 * through the interface the reference itself uses. Compiled together with the reference's own
 * src/backends/cpu_scalar/weight_resolve.c and src/formats/gguf/ sources, where they lie, into
 * oracle/_ref/libgeist_ref_wquant.so; this file only fills in a struct geist_weight
 * (include/geist_weight.h:133-151), lets cpu_scalar_resolve_weight pick the kernels
 * (weight_resolve.c:243-255) and calls them.
 */
#include <geist.h>
#include <geist_backend.h>
#include <geist_weight.h>

#include <stddef.h>

enum geist_status cpu_scalar_resolve_weight(struct geist_backend *be, struct geist_weight *w);

/* y[i][j] for m activation rows; dtype is the reference's enum geist_dtype value. Returns the
 * reference's status. */
int ref_wquant_linear(int dtype, const void *raw, int n_out, int n_in, const float *x, size_t m,
                      float *y) {
    struct geist_weight w = {0};
    w.raw                 = raw;
    w.n_in                = n_in;
    w.n_out               = n_out;
    w.dtype               = (uint16_t) dtype;
    const enum geist_status st = cpu_scalar_resolve_weight(nullptr, &w);
    if (st != GEIST_OK)
        return (int) st;
    if (m == 1)
        w.linear_m1(x, &w, nullptr, y);
    else
        w.linear_mN(x, &w, m, nullptr, y);
    return 0;
}

int ref_dtype_f16(void) { return (int) GEIST_DTYPE_F16; }
int ref_dtype_q6_K(void) { return (int) GEIST_DTYPE_Q6_K; }
int ref_dtype_q4_K(void) { return (int) GEIST_DTYPE_Q4_K; }
