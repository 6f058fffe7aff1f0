/*
 * lm_head.hip -- the two steps between the last transformer layer and the sampler
 * (src/archs/transformer/forward/head.c:94-129 of the reference), for gfx950:
 *
 *   k_rmsnorm_rows   cpu_scalar_rmsnorm               src/backends/cpu_scalar/elementwise.c:241-280
 *   k_f16_gemv       f16_gemv_m1 (tied F16 lm_head)   src/backends/cpu_x86/kernel_f16_gemv.c:34-64
 *
 * Both reproduce the reference's results bit for bit, which fixes the order of every sum.
 *
 * k_f16_gemv. The reference adds the products of a row in sixteen chains of fused multiply-adds
 * (two 8-lane AVX accumulators: element k belongs to chain k % 16 and is added at step k / 16),
 * then folds the chains in a fixed tree. A chain is sequential, so one lane owns eight chains of
 * one weight row -- the 16 bytes it needs per step are exactly one accumulator's 8 weights --
 * and two neighbouring lanes own a row. A wavefront therefore works on 32 rows at a time, and
 * reading 16 bytes per lane straight from those rows would touch 32 different lines per load.
 * Instead the wavefront streams the rows through a private LDS tile: it loads 128 bytes of each
 * of its 32 rows with fully coalesced 16-byte loads (8 lanes per row), two stages ahead in
 * registers, writes them to the tile (row pitch 144 bytes against bank conflicts), and each lane
 * reads its own 16 bytes per step back. No workgroup barrier is involved: the tile belongs to
 * one wavefront, whose LDS operations execute in order. The activations of the stage take the
 * same way (they come from L2). The kernel is bound by the one pass over the weights: 2 bytes
 * per multiply-add for one activation row, 2 / n_m bytes with n_m rows, whose accumulators
 * (8 per row and lane) share each converted weight.
 */
#include "lm_head_kernels.h"
#include "rmsnorm_device.h"

#include <hip/hip_fp16.h>

namespace gs {

namespace {

constexpr int LM_TPB       = 256;
constexpr int LM_WAVE      = 64;
constexpr int LM_WAVES     = LM_TPB / LM_WAVE;
constexpr int ROWS_WAVE    = 32;                   /* two lanes per weight row */
constexpr int ROWS_BLOCK   = ROWS_WAVE * LM_WAVES; /* 128 */
constexpr int STAGE_BYTES  = 128;                  /* of a row per stage */
constexpr int STAGE_COLS   = 64;                   /* ... which is 64 binary16 weights */
constexpr int STAGE_LOADS  = 4;                    /* 32 rows x 8 segments / 64 lanes */
constexpr int TILE_PITCH   = STAGE_BYTES + 16;     /* bytes */
constexpr int TILE_BYTES   = ROWS_WAVE * TILE_PITCH;
/* EB = bytes per weight: 2 (binary16) or 1 (int8 with a scale per row). A stage then holds
 * 128 / EB columns, 8 / EB steps of 16, and each lane stages 2 / EB activations per row. */
template <int EB>
struct Geom {
    static constexpr int COLS  = STAGE_BYTES / EB;
    static constexpr int STEPS = COLS / 16;
    static constexpr int XL    = COLS / LM_WAVE;
};

__device__ __forceinline__ float dadd(float a, float b) { return __fadd_rn(a, b); }

/* The weights of one stage for this lane: segment (lane & 7) of rows 8 i + (lane >> 3). */
struct StageRegs {
    uint4 w[STAGE_LOADS];
};

template <int MT, int XL>
struct StageX {
    float x[MT][XL];
};

/* Which weight row a wavefront's virtual row r (0..31) is. Plain: 32 consecutive rows per
 * wavefront task. Sampler layout: task (chunk, t) is thread t of chunk `chunk` of the sampler's
 * top-k scan (chunks of 8192 logits, thread t owns the float4 groups 4 * (j * 256 + t), j < 8),
 * so that the maximum over the task's 32 results is that thread's maximum. */
template <bool SL>
__device__ __forceinline__ long virtual_row(long task, int r) {
    if (!SL)
        return task * ROWS_WAVE + r;
    const long chunk = task >> 8, t = task & 255;
    return chunk * 8192 + 4 * ((long) (r >> 2) * 256 + t) + (r & 3);
}

template <int EB, bool SL>
__device__ __forceinline__ void stage_load(const uint8_t *__restrict__ w, long task, long n_out,
                                           int n_in, int stage, int lane, StageRegs &g) {
    const int seg = lane & 7;
    const int col = stage * Geom<EB>::COLS + seg * (16 / EB);
#pragma unroll
    for (int i = 0; i < STAGE_LOADS; ++i) {
        const long row = virtual_row<SL>(task, 8 * i + (lane >> 3));
        g.w[i]         = make_uint4(0u, 0u, 0u, 0u);
        if (row < n_out && col < n_in) {
            /* read once, and far more than the caches hold: non-temporal */
            typedef uint32_t nt_u4 __attribute__((ext_vector_type(4)));
            const nt_u4 t = __builtin_nontemporal_load(
                reinterpret_cast<const nt_u4 *>(w + (row * n_in + col) * EB));
            g.w[i] = make_uint4(t.x, t.y, t.z, t.w);
        }
    }
}

template <int EB, int MT>
__device__ __forceinline__ void stage_load_x(const float *__restrict__ x, long ld_x, int n_m,
                                             int n_in, int stage, int lane,
                                             StageX<MT, Geom<EB>::XL> &gx) {
#pragma unroll
    for (int q = 0; q < Geom<EB>::XL; ++q) {
        const int col = stage * Geom<EB>::COLS + q * LM_WAVE + lane;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int mm = m < n_m ? m : n_m - 1; /* rows beyond n_m repeat the last, unstored */
            gx.x[m][q]   = col < n_in ? x[mm * ld_x + col] : 0.0f;
        }
    }
}

/* One step of the chains: eight weights of this lane's row and half against the activations of
 * the same columns. MASKED: lanes with keep == false leave their chains alone. */
template <int EB, int MT, bool MASKED>
__device__ __forceinline__ void gemv_step(const uint8_t *tile, const float (*xs)[Geom<EB>::COLS],
                                          int my_row, int half, int t, bool keep,
                                          float (&acc)[MT][8]) {
    float wf[8];
    if (EB == 2) {
        const uint4 q =
            *reinterpret_cast<const uint4 *>(tile + my_row * TILE_PITCH + t * 32 + half * 16);
        const float2 f01 = __half22float2(*reinterpret_cast<const __half2 *>(&q.x));
        const float2 f23 = __half22float2(*reinterpret_cast<const __half2 *>(&q.y));
        const float2 f45 = __half22float2(*reinterpret_cast<const __half2 *>(&q.z));
        const float2 f67 = __half22float2(*reinterpret_cast<const __half2 *>(&q.w));
        wf[0] = f01.x, wf[1] = f01.y, wf[2] = f23.x, wf[3] = f23.y;
        wf[4] = f45.x, wf[5] = f45.y, wf[6] = f67.x, wf[7] = f67.y;
    } else {
        const uint2 q =
            *reinterpret_cast<const uint2 *>(tile + my_row * TILE_PITCH + t * 16 + half * 8);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            wf[i]     = (float) (int) (int8_t) (q.x >> (8 * i));
            wf[4 + i] = (float) (int) (int8_t) (q.y >> (8 * i));
        }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const float4 xa = *reinterpret_cast<const float4 *>(&xs[m][t * 16 + half * 8]);
        const float4 xb = *reinterpret_cast<const float4 *>(&xs[m][t * 16 + half * 8 + 4]);
        const float  xv[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float f = __builtin_fmaf(wf[i], xv[i], acc[m][i]);
            acc[m][i]     = (!MASKED || keep) ? f : acc[m][i];
        }
    }
}

/* The work of one workgroup; `scales` != NULL (int8 weights): y = sum * scales[row]. */
template <int EB, int MT, bool SL>
__device__ __forceinline__ void gemv_body(const uint8_t *__restrict__ w,
                                          const float *__restrict__ scales, long n_out, int n_in,
                                          const float *__restrict__ x, long ld_x, int n_m,
                                          float *__restrict__ y, long ld_y, const GemvFuse &fuse) {
    constexpr int COLS = Geom<EB>::COLS, STEPS = Geom<EB>::STEPS, XL = Geom<EB>::XL;
    __shared__ __align__(16) uint8_t s_tile[LM_WAVES][TILE_BYTES];
    __shared__ __align__(16) float   s_x[LM_WAVES][MT][COLS];
    const int  lane = threadIdx.x & (LM_WAVE - 1), wave = threadIdx.x / LM_WAVE;
    const long task = (long) blockIdx.x * LM_WAVES + wave;
    if (virtual_row<SL>(task, 0) >= n_out) { /* (no workgroup barrier below) */
        if (SL && lane < n_m && task < (long) fuse.n_chunks * 256)
            fuse.tmax[((long) lane * fuse.n_chunks + (task >> 8)) * 256 + (task & 255)] =
                __builtin_nanf(""); /* a scanning thread without an element is never chosen */
        return;
    }
    uint8_t *tile = s_tile[wave];
    float(*xs)[COLS] = s_x[wave];
    const int my_row = lane >> 1, half = lane & 1;

    float acc[MT][8];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int i = 0; i < 8; ++i)
            acc[m][i] = 0.0f;

    const int n_stage = (n_in + COLS - 1) / COLS;
    StageRegs      g0, g1;
    StageX<MT, XL> x0, x1;
    stage_load<EB, SL>(w, task, n_out, n_in, 0, lane, g0);
    if (n_stage > 1)
        stage_load<EB, SL>(w, task, n_out, n_in, 1, lane, g1);
    stage_load_x<EB, MT>(x, ld_x, n_m, n_in, 0, lane, x0);
    if (n_stage > 1)
        stage_load_x<EB, MT>(x, ld_x, n_m, n_in, 1, lane, x1);
    /* One stage: registers -> tile (this waits for the loads issued two stages ago), the same
     * registers are reloaded with the stage after next, then the steps. Two register sets take
     * turns, so nothing is copied. */
    auto do_stage = [&](int s, StageRegs &g, StageX<MT, XL> &gx) {
#pragma unroll
        for (int i = 0; i < STAGE_LOADS; ++i)
            *reinterpret_cast<uint4 *>(tile + (8 * i + (lane >> 3)) * TILE_PITCH + (lane & 7) * 16) =
                g.w[i];
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int q = 0; q < XL; ++q)
                xs[m][q * LM_WAVE + lane] = gx.x[m][q];
        if (s + 2 < n_stage) {
            stage_load<EB, SL>(w, task, n_out, n_in, s + 2, lane, g);
            stage_load_x<EB, MT>(x, ld_x, n_m, n_in, s + 2, lane, gx);
        }
        /* steps of this stage: whole blocks of 16 columns, and at the end of the row possibly
         * a block of 8, which only extends chains 0..7 (the lanes with half == 0) */
        const int left = n_in - s * COLS;
        if (left >= COLS) {
#pragma unroll
            for (int t = 0; t < STEPS; ++t)
                gemv_step<EB, MT, false>(tile, xs, my_row, half, t, true, acc);
        } else {
            const int  full  = left / 16;
            const bool tail8 = (left & 15) == 8;
            for (int t = 0; t < full; ++t)
                gemv_step<EB, MT, false>(tile, xs, my_row, half, t, true, acc);
            if (tail8)
                gemv_step<EB, MT, true>(tile, xs, my_row, half, full, half == 0, acc);
        }
    };
    for (int s = 0; s < n_stage; s += 2) {
        do_stage(s, g0, x0);
        if (s + 1 < n_stage)
            do_stage(s + 1, g1, x1);
    }
    /* (chain j + chain j+8), (lane i + lane i+4), ((0+1) + (2+3)): kernel_f16_gemv.c:25-32, 59 */
    const long row = virtual_row<SL>(task, my_row);
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
            v[i] = dadd(acc[m][i], __shfl_xor(acc[m][i], 1, LM_WAVE));
        const float q0 = dadd(v[0], v[4]), q1 = dadd(v[1], v[5]);
        const float q2 = dadd(v[2], v[6]), q3 = dadd(v[3], v[7]);
        float sum = dadd(dadd(q0, q1), dadd(q2, q3));
        if (EB == 1) /* q8w_gemv_m1: y[r] = s * scales[r], kernel_f16_gemv.c:125 */
            sum = __fmul_rn(sum, row < n_out ? scales[row] : 0.0f);
        if (half == 0 && row < n_out && m < n_m)
            y[m * ld_y + row] = sum;
        if (SL) {
            /* the scanning thread's maximum over its elements of the row (NaN ignored, as the
             * scan's v_max3_f32 does) */
            float mx = row < n_out ? sum : -__builtin_inff();
#pragma unroll
            for (int d = 1; d < LM_WAVE; d <<= 1)
                mx = __builtin_fmaxf(mx, __shfl_xor(mx, d, LM_WAVE));
            if (lane == 0 && m < n_m)
                fuse.tmax[((long) m * fuse.n_chunks + (task >> 8)) * 256 + (task & 255)] = mx;
        } else if (fuse.gmax != nullptr && m == 0) { /* (uniform) */
            float mx = row < n_out ? sum : -__builtin_inff();
#pragma unroll
            for (int d = 1; d < LM_WAVE; d <<= 1)
                mx = __builtin_fmaxf(mx, __shfl_xor(mx, d, LM_WAVE));
            if (lane == 0)
                fuse.gmax[task] = mx;
        }
    }
}

} // namespace

template <int MT, bool SL>
__global__ __launch_bounds__(LM_TPB) void k_f16_gemv(const uint16_t *__restrict__ w, long n_out,
                                                     int n_in, const float *__restrict__ x,
                                                     long ld_x, int n_m, float *__restrict__ y,
                                                     long ld_y, GemvFuse fuse) {
    gemv_body<2, MT, SL>(reinterpret_cast<const uint8_t *>(w), nullptr, n_out, n_in, x, ld_x, n_m,
                         y, ld_y, fuse);
}

/* q8w_gemv_m1 (kernel_f16_gemv.c:95-127): the same chains over int8 weights, times the row's
 * scale. Half the bytes per weight, so twice the columns per stage. */
template <int MT, bool SL>
__global__ __launch_bounds__(LM_TPB) void k_q8w_gemv(const int8_t *__restrict__ wq,
                                                     const float *__restrict__ scales, long n_out,
                                                     int n_in, const float *__restrict__ x,
                                                     long ld_x, int n_m, float *__restrict__ y,
                                                     long ld_y, GemvFuse fuse) {
    gemv_body<1, MT, SL>(reinterpret_cast<const uint8_t *>(wq), scales, n_out, n_in, x, ld_x, n_m,
                         y, ld_y, fuse);
}

/* The projection for several activation rows. Here a lane owns all sixteen chains of one weight
 * row (a wavefront works on 64 rows), so the activations of a step are the same for every lane
 * and come from scalar registers: each converted weight feeds n_m multiply-adds whose second
 * operand costs neither LDS traffic nor vector registers. The weights take the same way through
 * a private LDS tile as in k_f16_gemv. */
constexpr int ROWS_WAVE_B  = 64;
constexpr int ROWS_BLOCK_B = ROWS_WAVE_B * LM_WAVES;
constexpr int STAGE_LOADS_B = 8; /* 64 rows x 8 segments / 64 lanes */

struct StageRegsB {
    uint4 w[STAGE_LOADS_B];
};

__device__ __forceinline__ void stage_load_b(const uint16_t *__restrict__ w, long row0, long n_out,
                                             int n_in, int stage, int lane, StageRegsB &g) {
    const int col = stage * STAGE_COLS + (lane & 7) * 8;
#pragma unroll
    for (int i = 0; i < STAGE_LOADS_B; ++i) {
        const long row = row0 + 8 * i + (lane >> 3);
        g.w[i]         = make_uint4(0u, 0u, 0u, 0u);
        if (row < n_out && col < n_in) {
            typedef uint32_t nt_u4 __attribute__((ext_vector_type(4)));
            const nt_u4 t =
                __builtin_nontemporal_load(reinterpret_cast<const nt_u4 *>(w + row * n_in + col));
            g.w[i] = make_uint4(t.x, t.y, t.z, t.w);
        }
    }
}

/* Eight chains (one accumulator of the reference) of this lane's row against the activations
 * x[m][col .. col + 8), which are uniform over the wavefront. */
template <int MT>
__device__ __forceinline__ void gemv_half_step(const uint8_t *row_tile, int byte_off,
                                               const float *__restrict__ x, long ld_x, int n_m,
                                               int col, float (&acc)[MT][16], int chain0) {
    const uint4  q   = *reinterpret_cast<const uint4 *>(row_tile + byte_off);
    const float2 f01 = __half22float2(*reinterpret_cast<const __half2 *>(&q.x));
    const float2 f23 = __half22float2(*reinterpret_cast<const __half2 *>(&q.y));
    const float2 f45 = __half22float2(*reinterpret_cast<const __half2 *>(&q.z));
    const float2 f67 = __half22float2(*reinterpret_cast<const __half2 *>(&q.w));
    float        wf[8] = {f01.x, f01.y, f23.x, f23.y, f45.x, f45.y, f67.x, f67.y};
    /* keep the conversion a separate instruction: folded into a mixed-precision multiply-add it
     * is repeated per activation row, and that instruction takes no scalar operand, so every
     * activation would be copied to a vector register first */
#pragma unroll
    for (int i = 0; i < 8; ++i)
        asm("" : "+v"(wf[i]));
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const float *xm = x + (long) (m < n_m ? m : n_m - 1) * ld_x + col; /* uniform address */
#pragma unroll
        for (int i = 0; i < 8; ++i)
            acc[m][chain0 + i] = __builtin_fmaf(wf[i], xm[i], acc[m][chain0 + i]);
    }
}

template <int MT>
__global__ __launch_bounds__(LM_TPB) void k_f16_gemv_batched(const uint16_t *__restrict__ w,
                                                             long n_out, int n_in,
                                                             const float *__restrict__ x, long ld_x,
                                                             int n_m, float *__restrict__ y,
                                                             long ld_y) {
    __shared__ __align__(16) uint8_t s_tile[LM_WAVES][ROWS_WAVE_B * TILE_PITCH];
    const int  lane = threadIdx.x & (LM_WAVE - 1);
    const int  wave = __builtin_amdgcn_readfirstlane(threadIdx.x / LM_WAVE);
    const long row0 = (long) blockIdx.x * ROWS_BLOCK_B + wave * ROWS_WAVE_B;
    if (row0 >= n_out)
        return;
    uint8_t       *tile     = s_tile[wave];
    const uint8_t *row_tile = tile + lane * TILE_PITCH;

    float acc[MT][16];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int i = 0; i < 16; ++i)
            acc[m][i] = 0.0f;

    const int  n_stage = (n_in + STAGE_COLS - 1) / STAGE_COLS;
    StageRegsB g0, g1;
    stage_load_b(w, row0, n_out, n_in, 0, lane, g0);
    if (n_stage > 1)
        stage_load_b(w, row0, n_out, n_in, 1, lane, g1);
    for (int s = 0; s < n_stage; ++s) {
#pragma unroll
        for (int i = 0; i < STAGE_LOADS_B; ++i)
            *reinterpret_cast<uint4 *>(tile + (8 * i + (lane >> 3)) * TILE_PITCH + (lane & 7) * 16) =
                g0.w[i];
        g0 = g1;
        if (s + 2 < n_stage)
            stage_load_b(w, row0, n_out, n_in, s + 2, lane, g1);
        const int col0 = s * STAGE_COLS;
        const int left = n_in - col0;
        if (left >= STAGE_COLS) {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                gemv_half_step<MT>(row_tile, t * 32, x, ld_x, n_m, col0 + t * 16, acc, 0);
                gemv_half_step<MT>(row_tile, t * 32 + 16, x, ld_x, n_m, col0 + t * 16 + 8, acc, 8);
            }
        } else {
            const int full = left / 16;
            for (int t = 0; t < full; ++t) {
                gemv_half_step<MT>(row_tile, t * 32, x, ld_x, n_m, col0 + t * 16, acc, 0);
                gemv_half_step<MT>(row_tile, t * 32 + 16, x, ld_x, n_m, col0 + t * 16 + 8, acc, 8);
            }
            if ((left & 15) == 8) /* the block of eight extends chains 0..7 */
                gemv_half_step<MT>(row_tile, full * 32, x, ld_x, n_m, col0 + full * 16, acc, 0);
        }
    }
    const long row = row0 + lane;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
            v[i] = dadd(acc[m][i], acc[m][i + 8]);
        const float q0 = dadd(v[0], v[4]), q1 = dadd(v[1], v[5]);
        const float q2 = dadd(v[2], v[6]), q3 = dadd(v[3], v[7]);
        const float sum = dadd(dadd(q0, q1), dadd(q2, q3));
        if (row < n_out && m < n_m)
            y[m * ld_y + row] = sum;
    }
}

/* ---- the portable kernel's arithmetic: double accumulation -------------------------------- *
 * cpu_scalar_w_quant_m1 / _mN for F16 weights (src/backends/cpu_scalar/weight_resolve.c:186-241),
 * which the x86 backend also runs whenever more than one activation row is projected:
 *   y[i][j] = (float) sum_k (double) x[i][k] * (double) f16(W[j][k])   (double, index order).
 * Every product is exact in double (24 + 11 significant bits), so only the order of the
 * additions could differ from the reference, and that shows in the binary32 result only when
 * the sum lies within the additions' error of a binary32 rounding boundary. A lane owns a
 * weight row and adds in its own order (two partial sums per activation row); an output that
 * close to a boundary -- a few in a hundred thousand -- goes on a list, and a second kernel adds
 * those once more in index order, one lane per output. The error of either order is at most
 * n * 2^-53 times the largest partial sum on its way; the lane's two partial sums cover the
 * columns in ascending order, so after every stage of 64 columns |a0| + |a1| bounds both orders'
 * partial sums there, and within a stage a partial sum moves by at most ||w_stage|| ||x_stage||
 * (the weights' part is accumulated on the way in binary32, the activations' part comes with
 * their double copy). */

/* xd[m][k] = (double) x[m][k]; xs[m][s] = ||x[m][64 s .. 64 s + 63]||_2, rounded up; the count
 * of outputs left to the second kernel starts at zero. One workgroup per row, a wavefront per
 * stage of 64 columns. */
__global__ __launch_bounds__(LM_TPB) void k_x_to_f64(const float *__restrict__ x, long ld_x,
                                                     int n_in, double *__restrict__ xd,
                                                     double *__restrict__ xs, int *amb_count) {
    const int    lane = threadIdx.x & (LM_WAVE - 1), wave = threadIdx.x / LM_WAVE;
    const float *xr   = x + (long) blockIdx.x * ld_x;
    const int    n_stage = (n_in + STAGE_COLS - 1) / STAGE_COLS;
    if (blockIdx.x == 0 && threadIdx.x == 0)
        *amb_count = 0;
    for (int st = wave; st < n_stage; st += LM_WAVES) {
        const int k = st * STAGE_COLS + lane;
        double    v = 0.0;
        if (k < n_in) {
            v = (double) xr[k];
            xd[(long) blockIdx.x * n_in + k] = v;
        }
        double a = v * v;
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1)
            a += __shfl_xor(a, d, LM_WAVE);
        if (lane == 0)
            xs[(long) blockIdx.x * n_stage + st] = sqrt(a) * (1.0 + 0x1p-40);
    }
}

/* (float) s, and whether every value within err of s rounds to the same binary32. */
__device__ __forceinline__ bool f32_rounding_is_safe(double s, double err, float &f) {
    f = (float) s;
    if (!(__builtin_fabsf(f) < __builtin_inff()))
        return true; /* overflow or NaN: the order of the sum does not decide it */
    const double up = 0.5 * ((double) f + (double) nextafterf(f, __builtin_inff()));
    const double dn = 0.5 * ((double) f + (double) nextafterf(f, -__builtin_inff()));
    return up - s > err && s - dn > err;
}

/* One step of eight columns: this lane's weights against activations that are uniform over the
 * wavefront (scalar operands). */
template <int MT>
__device__ __forceinline__ void linear_f64_step(const uint8_t *row_tile, int byte_off,
                                                const double *__restrict__ xd, int n_in, int n_m,
                                                int col, double (&acc)[MT][2], float &w2) {
    const uint4  q   = *reinterpret_cast<const uint4 *>(row_tile + byte_off);
    const float2 f01 = __half22float2(*reinterpret_cast<const __half2 *>(&q.x));
    const float2 f23 = __half22float2(*reinterpret_cast<const __half2 *>(&q.y));
    const float2 f45 = __half22float2(*reinterpret_cast<const __half2 *>(&q.z));
    const float2 f67 = __half22float2(*reinterpret_cast<const __half2 *>(&q.w));
    const float  wf[8] = {f01.x, f01.y, f23.x, f23.y, f45.x, f45.y, f67.x, f67.y};
    double       wd[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        w2    = __builtin_fmaf(wf[i], wf[i], w2);
        wd[i] = (double) wf[i];
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const double *xm = xd + (long) (m < n_m ? m : n_m - 1) * n_in + col; /* uniform address */
#pragma unroll
        for (int i = 0; i < 8; ++i)
            acc[m][i & 1] = __builtin_fma(wd[i], xm[i], acc[m][i & 1]);
    }
}

template <int MT>
__global__ __launch_bounds__(LM_TPB) void k_f16_linear_f64(const uint16_t *__restrict__ w,
                                                           long n_out, int n_in,
                                                           const double *__restrict__ xd,
                                                           const double *__restrict__ xs, int n_m,
                                                           float *__restrict__ y, long ld_y,
                                                           int *__restrict__ amb_count,
                                                           int2 *__restrict__ amb_list) {
    __shared__ __align__(16) uint8_t s_tile[LM_WAVES][ROWS_WAVE_B * TILE_PITCH];
    const int  lane = threadIdx.x & (LM_WAVE - 1);
    const int  wave = __builtin_amdgcn_readfirstlane(threadIdx.x / LM_WAVE);
    const long row0 = (long) blockIdx.x * ROWS_BLOCK_B + wave * ROWS_WAVE_B;
    if (row0 >= n_out)
        return;
    uint8_t       *tile     = s_tile[wave];
    const uint8_t *row_tile = tile + lane * TILE_PITCH;

    double acc[MT][2], pmax[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
        acc[m][0] = acc[m][1] = pmax[m] = 0.0;

    const int  n_stage = (n_in + STAGE_COLS - 1) / STAGE_COLS;
    StageRegsB g0, g1;
    stage_load_b(w, row0, n_out, n_in, 0, lane, g0);
    if (n_stage > 1)
        stage_load_b(w, row0, n_out, n_in, 1, lane, g1);
    for (int s = 0; s < n_stage; ++s) {
#pragma unroll
        for (int i = 0; i < STAGE_LOADS_B; ++i)
            *reinterpret_cast<uint4 *>(tile + (8 * i + (lane >> 3)) * TILE_PITCH + (lane & 7) * 16) =
                g0.w[i];
        g0 = g1;
        if (s + 2 < n_stage)
            stage_load_b(w, row0, n_out, n_in, s + 2, lane, g1);
        const int col0 = s * STAGE_COLS;
        const int left = n_in - col0;
        double    p0[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m)
            p0[m] = fabs(acc[m][0]) + fabs(acc[m][1]);
        float w2 = 0.0f;
        if (left >= STAGE_COLS) {
#pragma unroll
            for (int t = 0; t < STAGE_COLS / 8; ++t)
                linear_f64_step<MT>(row_tile, t * 16, xd, n_in, n_m, col0 + t * 8, acc, w2);
        } else {
            for (int t = 0; t < left / 8; ++t)
                linear_f64_step<MT>(row_tile, t * 16, xd, n_in, n_m, col0 + t * 8, acc, w2);
        }
        /* ||w_stage||_2 from its binary32 sum of squares, rounded up by more than its error */
        const double wn = (double) __builtin_sqrtf(w2) * (1.0 + 1e-4);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const double p = p0[m] + wn * xs[(long) (m < n_m ? m : n_m - 1) * n_stage + s];
            pmax[m]        = p > pmax[m] ? p : pmax[m];
        }
    }
    const long row = row0 + lane;
    if (row >= n_out)
        return;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        if (m >= n_m)
            break;
        const double sum = acc[m][0] + acc[m][1];
        /* n 2^-53 (largest partial sum) for each of the two orders, and a little room for the
         * rounding of the bound itself */
        const double err = (double) n_in * 0x1p-52 * 1.01 * pmax[m];
        float        f;
        if (!f32_rounding_is_safe(sum, err, f))
            amb_list[atomicAdd(amb_count, 1)] = make_int2((int) row, m);
        y[m * ld_y + row] = f;
    }
}

/* The same projection for 5 to 16 activation rows on the double-precision matrix cores. A
 * wavefront owns 64 weight rows (four tiles of 16) against up to 16 activation rows; one
 * v_mfma_f64_16x16x4 adds four columns to a 16 x 16 tile: A = activations [m][k], B = weights
 * [k][row], lane l holds A[l % 16][l / 16] and B[l / 16][l % 16], and of the result the rows
 * l / 16, 4 + l / 16, 8 + l / 16, 12 + l / 16 of column l % 16. Within a stage of 64 columns instruction t takes
 * the columns t, 16 + t, 32 + t, 48 + t, so that a lane converts 16 consecutive weights of its
 * row and reads 16 consecutive activations. The order inside a stage is therefore not the
 * reference's either; the bound and the list are those of the vector kernel (partial sums are
 * sampled at the stage boundaries, where all earlier columns have been added; the room for the
 * error is doubled for the matrix cores' internal additions).
 * NS > 0 (2 to 12 activation rows): v_mfma_f64_4x4x4 instead, four independent 4 x 4 x 4 blocks
 * per instruction, NS instructions for NS sets of four activation rows. Lane l holds A[l % 4][l / 16] of block (l / 4) % 4 -- the activations, the same
 * in every block --, B[l / 16][l % 4] of that block -- weight row l % 16 of the tile, as above --
 * and the result of activation row l / 16 (of its set) and weight row l % 16. A quarter of the
 * arithmetic per set for the same pass over the weights. */
typedef double mfma_d4 __attribute__((ext_vector_type(4)));

template <int NS>
__global__ __launch_bounds__(LM_TPB, 2) void k_f16_linear_f64_mfma(
    const uint16_t *__restrict__ w, long n_out, int n_in, const double *__restrict__ xd,
    const double *__restrict__ xs, int n_m, float *__restrict__ y, long ld_y,
    int *__restrict__ amb_count, int2 *__restrict__ amb_list) {
    __shared__ __align__(16) uint8_t s_tile[LM_WAVES][ROWS_WAVE_B * TILE_PITCH];
    /* the activations of a stage, for the whole workgroup, two stages alternating (rows two
     * doubles apart in the banks) */
    __shared__ __align__(16) double s_xa[2][F64_M_MAX][STAGE_COLS + 2];
    const int  lane = threadIdx.x & (LM_WAVE - 1);
    const int  wave = __builtin_amdgcn_readfirstlane(threadIdx.x / LM_WAVE);
    const long row0 = (long) blockIdx.x * ROWS_BLOCK_B + wave * ROWS_WAVE_B;
    /* (a wavefront without rows stays for the workgroup's barriers; its loads are masked) */
    uint8_t  *tile = s_tile[wave];
    const int j = lane & 15, kq = lane >> 4;
    /* this thread's share of a stage's activations: four columns of row tid / 16 */
    const int     xl_row = (int) threadIdx.x >> 4, xl_col = ((int) threadIdx.x & 15) * 4;
    const double *xl_src = xd + (long) (xl_row < n_m ? xl_row : 0) * n_in + xl_col;
    auto load_x = [&](int s, double (&xr)[4]) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int c = s * STAGE_COLS + xl_col + q;
            xr[q]       = (xl_row < n_m && c < n_in) ? xl_src[s * STAGE_COLS + q] : 0.0;
        }
    };
    auto store_x = [&](int buf, const double (&xr)[4]) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
            s_xa[buf][xl_row][xl_col + q] = xr[q];
    };

    /* NS == 0: one 16 x 16 x 4 instruction per four columns; NS > 0: NS instructions of four
     * 4 x 4 x 4 blocks, set q for the activation rows 4 q .. 4 q + 3. Either way a lane holds,
     * per tile of 16 weight rows, the results of the activation rows 4 r + kq. */
    constexpr bool SMALL = NS > 0;
    constexpr int  NR = SMALL ? NS : 4, NA = SMALL ? NS : 1;
    const int      ja = SMALL ? (lane & 3) : j; /* the activation row this lane feeds as A (+ 4 q) */
    mfma_d4 acc[4];
    double  pmax[4][NR];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        acc[t] = mfma_d4{0.0, 0.0, 0.0, 0.0};
#pragma unroll
        for (int r = 0; r < NR; ++r)
            pmax[t][r] = 0.0;
    }
    const int  n_stage = (n_in + STAGE_COLS - 1) / STAGE_COLS;
    StageRegsB g0, g1;
    stage_load_b(w, row0, n_out, n_in, 0, lane, g0);
    if (n_stage > 1)
        stage_load_b(w, row0, n_out, n_in, 1, lane, g1);
    {
        double xr[4];
        load_x(0, xr);
        store_x(0, xr);
    }
    __syncthreads();
    for (int s = 0; s < n_stage; ++s) {
        /* the next stage's activations are requested now and stored at the end of this stage */
        double xnext[4];
        if (s + 1 < n_stage)
            load_x(s + 1, xnext);
        /* (activations of the stage: columns 16 kq .. 16 kq + 15 of row ja + 4 q, read below) */
        double xst[NR]; /* ||x_stage|| of the activation rows this lane holds results of */
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int m = 4 * r + kq;
            xst[r]      = xs[(long) (m < n_m ? m : n_m - 1) * n_stage + s];
        }
#pragma unroll
        for (int i = 0; i < STAGE_LOADS_B; ++i)
            *reinterpret_cast<uint4 *>(tile + (8 * i + (lane >> 3)) * TILE_PITCH + (lane & 7) * 16) =
                g0.w[i];
        g0 = g1;
        if (s + 2 < n_stage)
            stage_load_b(w, row0, n_out, n_in, s + 2, lane, g1);
        /* the four tiles' instructions interleaved: consecutive ones do not wait for each other */
        uint32_t u[4][8];
        float    w2[4];
#pragma unroll
        for (int tl = 0; tl < 4; ++tl) {
            const uint8_t *src = tile + (16 * tl + j) * TILE_PITCH + kq * 32;
            const uint4    qa  = *reinterpret_cast<const uint4 *>(src);
            const uint4    qb  = *reinterpret_cast<const uint4 *>(src + 16);
            u[tl][0] = qa.x, u[tl][1] = qa.y, u[tl][2] = qa.z, u[tl][3] = qa.w;
            u[tl][4] = qb.x, u[tl][5] = qb.y, u[tl][6] = qb.z, u[tl][7] = qb.w;
            w2[tl] = 0.0f;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            double2 xv[NA];
#pragma unroll
            for (int q = 0; q < NA; ++q)
                xv[q] = *reinterpret_cast<const double2 *>(&s_xa[s & 1][ja + 4 * q][16 * kq + 2 * i]);
#pragma unroll
            for (int tl = 0; tl < 4; ++tl) {
                const float2 f = __half22float2(*reinterpret_cast<const __half2 *>(&u[tl][i]));
                w2[tl]         = __builtin_fmaf(f.x, f.x, w2[tl]);
                w2[tl]         = __builtin_fmaf(f.y, f.y, w2[tl]);
                const double wd = (double) f.x;
                if (SMALL) {
#pragma unroll
                    for (int q = 0; q < NA; ++q)
                        acc[tl][q] = __builtin_amdgcn_mfma_f64_4x4x4f64(xv[q].x, wd, acc[tl][q], 0, 0, 0);
                } else {
                    acc[tl] = __builtin_amdgcn_mfma_f64_16x16x4f64(xv[0].x, wd, acc[tl], 0, 0, 0);
                }
            }
#pragma unroll
            for (int tl = 0; tl < 4; ++tl) {
                const float2 f = __half22float2(*reinterpret_cast<const __half2 *>(&u[tl][i]));
                const double wd = (double) f.y;
                if (SMALL) {
#pragma unroll
                    for (int q = 0; q < NA; ++q)
                        acc[tl][q] = __builtin_amdgcn_mfma_f64_4x4x4f64(xv[q].y, wd, acc[tl][q], 0, 0, 0);
                } else {
                    acc[tl] = __builtin_amdgcn_mfma_f64_16x16x4f64(xv[0].y, wd, acc[tl], 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (int tl = 0; tl < 4; ++tl) {
            /* ||w_stage|| of row j: the four lanes j, j + 16, j + 32, j + 48 hold a quarter each */
            float ws2 = w2[tl];
            ws2 += __shfl_xor(ws2, 16, LM_WAVE);
            ws2 += __shfl_xor(ws2, 32, LM_WAVE);
            const double wn = (double) __builtin_sqrtf(ws2) * (1.0 + 1e-4);
#pragma unroll
            for (int r = 0; r < NR; ++r) {
                /* (a partial sum inside the stage differs from the one at its end by at most
                 * the stage's ||w|| ||x||, as from the one at its start) */
                const double p = fabs(acc[tl][r]) + wn * xst[r];
                pmax[tl][r]    = p > pmax[tl][r] ? p : pmax[tl][r];
            }
        }
        if (s + 1 < n_stage)
            store_x((s + 1) & 1, xnext);
        __syncthreads();
    }
#pragma unroll
    for (int tl = 0; tl < 4; ++tl) {
        const long row = row0 + 16 * tl + j;
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int m = 4 * r + kq;
            if (row >= n_out || m >= n_m)
                continue;
            const double sum = acc[tl][r];
            const double err = (double) n_in * 0x1p-51 * 1.01 * pmax[tl][r];
            float        f;
            if (!f32_rounding_is_safe(sum, err, f))
                amb_list[atomicAdd(amb_count, 1)] = make_int2((int) row, m);
            y[m * ld_y + row] = f;
        }
    }
}

/* The listed outputs once more, the products added one after the other in index order as the
 * reference adds them. A wavefront per output (weight row r, activation row m): its lanes form
 * 256 products at a time -- each exact in double -- and put them into the wavefront's part of
 * LDS; the sum then takes them in order, two per 16-byte read that every lane makes of the same
 * address. The chain of n_in dependent additions is what this kernel takes (a wavefront issues
 * an instruction every few cycles whatever it is: 1.5 instructions per product here, where
 * fetching each product from its lane as a scalar operand took three); there are few listed
 * outputs and each has a wavefront to itself. */
__global__ __launch_bounds__(LM_TPB) void k_f16_linear_f64_listed(
    const uint16_t *__restrict__ w, int n_in, const double *__restrict__ xd, float *__restrict__ y,
    long ld_y, const int *__restrict__ amb_count, const int2 *__restrict__ amb_list) {
    __shared__ __align__(16) double s_prod[LM_WAVES][4 * LM_WAVE];
    const int lane = threadIdx.x & (LM_WAVE - 1), wave = threadIdx.x / LM_WAVE;
    double   *mine_p = s_prod[wave];
    const int count = *amb_count;
    for (int it = (int) blockIdx.x * LM_WAVES + wave; it < count;
         it += (int) gridDim.x * LM_WAVES) { /* (uniform over the wavefront) */
        const int2      mine = amb_list[it];
        const uint16_t *wr   = w + (long) mine.x * n_in;
        const double   *xm   = xd + (long) mine.y * n_in;
        double          acc  = 0.0;
        for (int k0 = 0; k0 < n_in; k0 += 4 * LM_WAVE) {
            /* four rounds of 64 products, their loads in flight together; a short last round
             * adds zeros, which change nothing (the sum never is -0 after a +0 start) */
            double prod[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int k = k0 + r * LM_WAVE + lane;
                prod[r]     = k < n_in ? xm[k] * (double) __half2float(__ushort_as_half(wr[k])) : 0.0;
            }
            /* (the wavefront's own reads of the block before are done: its LDS operations are
             * performed in the order they were issued) */
#pragma unroll
            for (int r = 0; r < 4; ++r)
                mine_p[r * LM_WAVE + lane] = prod[r];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            const int n_here = n_in - k0 < 4 * LM_WAVE ? n_in - k0 : 4 * LM_WAVE;
            const int pairs  = (n_here + 1) >> 1; /* (an odd count ends with a zero) */
            const double2 *pp = reinterpret_cast<const double2 *>(mine_p);
#pragma unroll 16
            for (int i = 0; i < pairs; ++i) {
                const double2 t = pp[i];
                acc += t.x;
                acc += t.y;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
        if (lane == 0)
            y[mine.y * ld_y + mine.x] = (float) acc;
    }
}

/* One workgroup per row. The reference adds the squares in double in index order; the order of
 * a double sum only shows in the binary32 result when 1 / sqrt(mean + eps) lies within the
 * sum's error of the middle between two binary32 values. The workgroup adds in a fixed parallel
 * order and, in that rare case, one thread repeats the sum in the reference's order. */
__global__ __launch_bounds__(LM_TPB) void k_rmsnorm_rows(const float *__restrict__ x, long ld_x,
                                                         const float *__restrict__ w, float eps,
                                                         int n, float *__restrict__ y, long ld_y) {
    __shared__ double s_part[LM_TPB];
    __shared__ float  s_inv;
    const int    tid = threadIdx.x;
    const float *xr  = x + (long) blockIdx.x * ld_x;
    float       *yr  = y + (long) blockIdx.x * ld_y;
    const float inv = block_rms_inv<LM_TPB>(xr, n, eps, s_part, &s_inv);
    for (int i = tid; i < n; i += LM_TPB)
        yr[i] = __fmul_rn(__fmul_rn(xr[i], inv), w[i]);
}

void launch_rmsnorm_rows(hipStream_t stream, const float *x, long ld_x, const float *w, float eps,
                         int n_rows, int n, float *y, long ld_y) {
    k_rmsnorm_rows<<<dim3(n_rows), dim3(LM_TPB), 0, stream>>>(x, ld_x, w, eps, n, y, ld_y);
}

bool f16_gemv_can_fuse(int n_m) { return n_m >= 1 && n_m <= 2; }

void launch_f16_gemv(hipStream_t stream, const uint16_t *w_f16, long n_out, int n_in,
                     const float *x, long ld_x, int n_m, float *y, long ld_y,
                     const GemvFuse *fuse) {
    const dim3 block(LM_TPB);
    const dim3 grid((unsigned) ((n_out + ROWS_BLOCK - 1) / ROWS_BLOCK));
    const dim3 grid_b((unsigned) ((n_out + ROWS_BLOCK_B - 1) / ROWS_BLOCK_B));
    GemvFuse   none{};
    if (fuse && fuse->tmax) { /* (the caller has asked f16_gemv_can_fuse) */
        const dim3 grid_s((unsigned) (fuse->n_chunks * 256 / LM_WAVES));
        if (n_m <= 1)
            k_f16_gemv<1, true><<<grid_s, block, 0, stream>>>(w_f16, n_out, n_in, x, ld_x, n_m, y, ld_y, *fuse);
        else
            k_f16_gemv<2, true><<<grid_s, block, 0, stream>>>(w_f16, n_out, n_in, x, ld_x, n_m, y, ld_y, *fuse);
        return;
    }
    if (n_m <= 1)
        k_f16_gemv<1, false><<<grid, block, 0, stream>>>(w_f16, n_out, n_in, x, ld_x, n_m, y, ld_y, none);
    else if (n_m <= 2)
        k_f16_gemv<2, false><<<grid, block, 0, stream>>>(w_f16, n_out, n_in, x, ld_x, n_m, y, ld_y, none);
    else if (n_m <= 4) /* (with 8 rows the batched kernel's 128 accumulators leave no room) */
        k_f16_gemv_batched<4><<<grid_b, block, 0, stream>>>(w_f16, n_out, n_in, x, ld_x, n_m, y, ld_y);
    else
        k_f16_gemv<8, false><<<grid, block, 0, stream>>>(w_f16, n_out, n_in, x, ld_x, n_m, y, ld_y, none);
}

void launch_f16_linear_f64(hipStream_t stream, const uint16_t *w_f16, long n_out, int n_in,
                           const float *x, long ld_x, int n_m, const F64Scratch &ws, float *y,
                           long ld_y) {
    const dim3 block(LM_TPB);
    const dim3 grid_b((unsigned) ((n_out + ROWS_BLOCK_B - 1) / ROWS_BLOCK_B));
    k_x_to_f64<<<dim3(n_m), block, 0, stream>>>(x, ld_x, n_in, ws.xd, ws.xs, ws.amb_count);
    if (n_m <= 1)
        k_f16_linear_f64<1><<<grid_b, block, 0, stream>>>(w_f16, n_out, n_in, ws.xd, ws.xs, n_m, y, ld_y, ws.amb_count, ws.amb_list);
    else if (n_m <= 4) /* four 4 x 4 x 4 blocks per matrix-core instruction */
        k_f16_linear_f64_mfma<1><<<grid_b, block, 0, stream>>>(w_f16, n_out, n_in, ws.xd, ws.xs, n_m, y, ld_y, ws.amb_count, ws.amb_list);
    else if (n_m <= 8) /* ... two such instructions, for the rows 0..3 and 4..7 */
        k_f16_linear_f64_mfma<2><<<grid_b, block, 0, stream>>>(w_f16, n_out, n_in, ws.xd, ws.xs, n_m, y, ld_y, ws.amb_count, ws.amb_list);
    else if (n_m <= 12)
        k_f16_linear_f64_mfma<3><<<grid_b, block, 0, stream>>>(w_f16, n_out, n_in, ws.xd, ws.xs, n_m, y, ld_y, ws.amb_count, ws.amb_list);
    else /* 13 .. F64_M_MAX rows: one 16 x 16 tile of activation rows */
        k_f16_linear_f64_mfma<0><<<grid_b, block, 0, stream>>>(w_f16, n_out, n_in, ws.xd, ws.xs, n_m, y, ld_y, ws.amb_count, ws.amb_list);
    /* normally a few dozen outputs, whose number is only known on the device: a wavefront for
     * up to one output in 256, most of which return at once; longer lists go round the loop */
    const long     want_wgs   = (n_out * n_m / 256 + LM_WAVES - 1) / LM_WAVES + 1;
    const unsigned listed_wgs = (unsigned) (want_wgs < 2048 ? want_wgs : 2048);
    k_f16_linear_f64_listed<<<dim3(listed_wgs), block, 0, stream>>>(w_f16, n_in, ws.xd, y, ld_y,
                                                                   ws.amb_count, ws.amb_list);
}

/* f16_to_q8w (kernel_f16_gemv.c:66-93): per row scale = max|w| / 127, q = lrintf(w * (127 /
 * max|w|)) clamped to +-127. One workgroup per row. */
__global__ __launch_bounds__(LM_TPB) void k_f16_to_q8w(const uint16_t *__restrict__ w, int n_in,
                                                       int8_t *__restrict__ wq,
                                                       float *__restrict__ scales) {
    __shared__ float s_max[LM_TPB];
    const int        tid = threadIdx.x;
    const uint16_t  *wr  = w + (long) blockIdx.x * n_in;
    float            a   = 0.0f;
    for (int k = tid; k < n_in; k += LM_TPB) {
        const float v = fabsf(__half2float(*reinterpret_cast<const __half *>(wr + k)));
        a             = v > a ? v : a; /* (a NaN never replaces the maximum, as in the reference) */
    }
    s_max[tid] = a;
    __syncthreads();
    for (int step = LM_TPB / 2; step > 0; step >>= 1) {
        if (tid < step)
            s_max[tid] = s_max[tid + step] > s_max[tid] ? s_max[tid + step] : s_max[tid];
        __syncthreads();
    }
    const float amax = s_max[0];
    const float id   = amax > 0.0f ? __fdiv_rn(127.0f, amax) : 0.0f;
    if (tid == 0)
        scales[blockIdx.x] = __fdiv_rn(amax, 127.0f);
    int8_t *qr = wq + (long) blockIdx.x * n_in;
    for (int k = tid; k < n_in; k += LM_TPB) {
        const float v = __fmul_rn(__half2float(*reinterpret_cast<const __half *>(wr + k)), id);
        int         q = __float2int_rn(v); /* lrintf: to nearest, ties to even */
        q             = q > 127 ? 127 : q;
        q             = q < -127 ? -127 : q;
        qr[k]         = (int8_t) q;
    }
}

void launch_f16_to_q8w(hipStream_t stream, const uint16_t *w_f16, long n_out, int n_in, int8_t *wq,
                       float *scales) {
    k_f16_to_q8w<<<dim3((unsigned) n_out), dim3(LM_TPB), 0, stream>>>(w_f16, n_in, wq, scales);
}

void launch_q8w_gemv(hipStream_t stream, const int8_t *wq, const float *scales, long n_out,
                     int n_in, const float *x, long ld_x, int n_m, float *y, long ld_y,
                     const GemvFuse *fuse) {
    const dim3 block(LM_TPB);
    const dim3 grid((unsigned) ((n_out + ROWS_BLOCK - 1) / ROWS_BLOCK));
    GemvFuse   none{};
    if (fuse && fuse->tmax) {
        const dim3 grid_s((unsigned) (fuse->n_chunks * 256 / LM_WAVES));
        if (n_m <= 1)
            k_q8w_gemv<1, true><<<grid_s, block, 0, stream>>>(wq, scales, n_out, n_in, x, ld_x, n_m, y, ld_y, *fuse);
        else
            k_q8w_gemv<2, true><<<grid_s, block, 0, stream>>>(wq, scales, n_out, n_in, x, ld_x, n_m, y, ld_y, *fuse);
        return;
    }
    if (n_m <= 1)
        k_q8w_gemv<1, false><<<grid, block, 0, stream>>>(wq, scales, n_out, n_in, x, ld_x, n_m, y, ld_y,
                                                         fuse ? *fuse : none);
    else if (n_m <= 2)
        k_q8w_gemv<2, false><<<grid, block, 0, stream>>>(wq, scales, n_out, n_in, x, ld_x, n_m, y, ld_y, none);
    else if (n_m <= 4)
        k_q8w_gemv<4, false><<<grid, block, 0, stream>>>(wq, scales, n_out, n_in, x, ld_x, n_m, y, ld_y, none);
    else
        k_q8w_gemv<8, false><<<grid, block, 0, stream>>>(wq, scales, n_out, n_in, x, ld_x, n_m, y, ld_y, none);
}

} // namespace gs
