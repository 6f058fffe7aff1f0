/* Device helpers of the output RMS norm (cpu_scalar_rmsnorm,
 * src/backends/cpu_scalar/elementwise.c:241-280), shared by the kernels that norm a hidden row. */
#ifndef GEIST_RMSNORM_DEVICE_H
#define GEIST_RMSNORM_DEVICE_H

#include <hip/hip_runtime.h>

namespace gs {

/* 1 / sqrt(mean(x^2) + eps) as cpu_scalar_rmsnorm rounds it (elementwise.c:270-274). The
 * reference adds the squares in double in index order; the order of a double sum only shows in
 * the binary32 result when the value lies within the sums' error of the middle between two
 * binary32 values, and then `sequential` repeats the sum in the reference's order. */
__device__ __forceinline__ bool rms_inv_is_safe(double sumsq, int n, float eps, float &f) {
    const double r  = 1.0 / sqrt(sumsq / (double) n + (double) eps);
    f               = (float) r;
    const float  fn = r > (double) f ? nextafterf(f, __builtin_inff()) : nextafterf(f, -__builtin_inff());
    const double mid = 0.5 * ((double) f + (double) fn);
    return !(fabs(r - mid) <= fabs(r) * (double) n * 0x1p-50);
}
__device__ __forceinline__ float rms_inv_sequential(const float *__restrict__ xr, int n, float eps) {
    double sumsq = 0.0;
    for (int i = 0; i < n; ++i)
        sumsq += (double) xr[i] * (double) xr[i];
    return (float) (1.0 / sqrt(sumsq / (double) n + (double) eps));
}

/* The inverse RMS of xr[0..n) for a workgroup of TPB threads, every thread gets it: the squares
 * are added in double in a fixed parallel order (thread t takes the elements t, t + TPB, ...,
 * then a binary tree over the threads) and, where the binary32 result could depend on the
 * order, once more by one thread in the reference's order. s_part is [TPB], s_inv one float. */
template <int TPB>
__device__ __forceinline__ float block_rms_inv(const float *__restrict__ xr, int n, float eps,
                                               double *s_part, float *s_inv) {
    const int tid = threadIdx.x;
    double    a   = 0.0;
    for (int i = tid; i < n; i += TPB)
        a += (double) xr[i] * (double) xr[i];
    s_part[tid] = a;
    __syncthreads();
    for (int step = TPB / 2; step > 0; step >>= 1) {
        if (tid < step)
            s_part[tid] += s_part[tid + step];
        __syncthreads();
    }
    if (tid == 0) {
        float f;
        if (!rms_inv_is_safe(s_part[0], n, eps, f))
            f = rms_inv_sequential(xr, n, eps);
        *s_inv = f;
    }
    __syncthreads();
    return *s_inv;
}

} // namespace gs
#endif
