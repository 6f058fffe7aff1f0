/*
 * sampler_device.h -- device-side building blocks shared by the sampling kernels (gfx950,
 * wavefront 64, 256-thread workgroups).
 *
 * Layout of a logit row in a launch: the row is cut into n_chunks pieces of `per_chunk`
 * elements (a multiple of 64 floats, so every chunk starts on a 256-byte boundary of the row).
 * One workgroup owns one (row, chunk) pair and holds the whole chunk in registers: thread t
 * owns the float4 groups f = j * 256 + t, j = 0 .. NV-1, i.e. a wavefront reads 1 KiB of
 * consecutive addresses per load instruction.
 */
#ifndef GEIST_SAMPLER_DEVICE_H
#define GEIST_SAMPLER_DEVICE_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "glibc_expf.h"
#include "glibc_tanhf.h"
#include "sampler_kernels.h"

namespace gs {

constexpr int TPB    = 256;
constexpr int WAVE   = 64;
constexpr int NWAVES = TPB / WAVE;

/* Order-preserving map fp32 -> u32 used for every comparison on this path. It restates the
 * reference's comparisons (src/engine/sampler.c:56, 72, 171-174): -0 and +0 are equal, and a
 * NaN never compares greater, so it takes the lowest key. */
__device__ __forceinline__ uint32_t f2key(float x) {
    uint32_t b = __float_as_uint(x);
    if (x != x)
        return 0u;
    if ((b << 1) == 0u)
        b = 0u;
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float key2f(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

/* (key, index) packed so that an unsigned max picks the greater key and, among equal keys,
 * the LOWER index (src/engine/sampler.c:56: strict '>' keeps the first maximum). */
__device__ __forceinline__ uint64_t pack_best(uint32_t key, uint32_t idx) {
    return ((uint64_t) key << 32) | (uint64_t) (0xffffffffu - idx);
}
__device__ __forceinline__ uint32_t best_idx(uint64_t p) { return 0xffffffffu - (uint32_t) p; }
__device__ __forceinline__ uint32_t best_key(uint64_t p) { return (uint32_t) (p >> 32); }

/* Workgroup barrier that orders LDS traffic only. __syncthreads() also waits for every global
 * load in flight (its fence covers all address spaces); where loads should stay outstanding
 * across the barrier -- the chunk's logits while the history table is built -- this one waits
 * for the LDS counter alone. */
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

/* ---- wavefront-64 reductions -------------------------------------------------------------- */
/* All by DPP moves (shifts inside each row of 16 lanes, then the row results are broadcast into
 * the following rows), so that lane 63 ends with the result over all 64 lanes; a readlane hands
 * it to every lane. No LDS crossbar traffic, and a fixed order of combination. Lanes without a
 * source receive 0, the neutral element of every reduction here. */
__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int m) {
    uint32_t lo = (uint32_t) v, hi = (uint32_t) (v >> 32);
    lo = (uint32_t) __shfl_xor((int) lo, m, WAVE);
    hi = (uint32_t) __shfl_xor((int) hi, m, WAVE);
    return ((uint64_t) hi << 32) | lo;
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_fetch_u32(uint32_t v) {
    return (uint32_t) __builtin_amdgcn_update_dpp(0, (int) v, CTRL, ROW_MASK, 0xf, false);
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint64_t dpp_fetch_u64(uint64_t v) {
    return ((uint64_t) dpp_fetch_u32<CTRL, ROW_MASK>((uint32_t) (v >> 32)) << 32) |
           dpp_fetch_u32<CTRL, ROW_MASK>((uint32_t) v);
}
__device__ __forceinline__ uint32_t readlane_u32(uint32_t v, int lane) {
    return (uint32_t) __builtin_amdgcn_readlane((int) v, lane);
}
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
#define GS_STEP(ctrl, rows)                                                                    \
    {                                                                                          \
        const uint64_t o = dpp_fetch_u64<ctrl, rows>(v);                                       \
        v                = o > v ? o : v;                                                      \
    }
    GS_STEP(0x111, 0xf) GS_STEP(0x112, 0xf) GS_STEP(0x114, 0xf) GS_STEP(0x118, 0xf)
    GS_STEP(0x142, 0xa) GS_STEP(0x143, 0xc)
#undef GS_STEP
    return ((uint64_t) readlane_u32((uint32_t) (v >> 32), WAVE - 1) << 32) |
           readlane_u32((uint32_t) v, WAVE - 1);
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#define GS_STEP(ctrl, rows)                                                                    \
    {                                                                                          \
        const uint32_t o = dpp_fetch_u32<ctrl, rows>(v);                                       \
        v                = o > v ? o : v;                                                      \
    }
    GS_STEP(0x111, 0xf) GS_STEP(0x112, 0xf) GS_STEP(0x114, 0xf) GS_STEP(0x118, 0xf)
    GS_STEP(0x142, 0xa) GS_STEP(0x143, 0xc)
#undef GS_STEP
    return readlane_u32(v, WAVE - 1);
}
__device__ __forceinline__ double wave_scan_f64_dpp(double v);
__device__ __forceinline__ int    wave_scan_i32_dpp(int v);
__device__ __forceinline__ double wave_sum_f64(double v) {
    const uint64_t t = (uint64_t) __double_as_longlong(wave_scan_f64_dpp(v));
    return __longlong_as_double((long long) (((uint64_t) readlane_u32((uint32_t) (t >> 32), WAVE - 1) << 32) |
                                             readlane_u32((uint32_t) t, WAVE - 1)));
}
/* inclusive prefix sums over the lanes of a wavefront, lane order */
__device__ __forceinline__ double wave_scan_f64(double v) { return wave_scan_f64_dpp(v); }
__device__ __forceinline__ int    wave_scan_i32(int v) { return wave_scan_i32_dpp(v); }

/* Inclusive prefix sum over the wavefront with DPP moves: shifts inside each row of 16 lanes,
 * then the row totals are broadcast into the following rows. */
__device__ __forceinline__ int wave_scan_i32_dpp(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false); /* row_shr:1 */
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false); /* row_shr:2 */
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false); /* row_shr:4 */
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false); /* row_shr:8 */
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false); /* row_bcast:15 -> rows 1, 3 */
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false); /* row_bcast:31 -> rows 2, 3 */
    return v;
}
/* Sum of a float over the wavefront by the same DPP steps; every lane receives the total
 * (the order of the additions is fixed, so equal inputs give equal sums). */
__device__ __forceinline__ float wave_sum_f32_dpp(float v) {
#define GS_DPP_F32(ctrl, rows) \
    __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, rows, 0xf, false))
    v += GS_DPP_F32(0x111, 0xf);
    v += GS_DPP_F32(0x112, 0xf);
    v += GS_DPP_F32(0x114, 0xf);
    v += GS_DPP_F32(0x118, 0xf);
    v += GS_DPP_F32(0x142, 0xa);
    v += GS_DPP_F32(0x143, 0xc);
#undef GS_DPP_F32
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), WAVE - 1));
}
/* The same for doubles: both halves travel by DPP, lanes without a source add 0.0. */
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_fetch_f64(double v) {
    const uint64_t u  = (uint64_t) __double_as_longlong(v);
    const int      lo = __builtin_amdgcn_update_dpp(0, (int) (uint32_t) u, CTRL, ROW_MASK, 0xf, false);
    const int      hi =
        __builtin_amdgcn_update_dpp(0, (int) (uint32_t) (u >> 32), CTRL, ROW_MASK, 0xf, false);
    return __longlong_as_double((long long) (((uint64_t) (uint32_t) hi << 32) | (uint32_t) lo));
}
__device__ __forceinline__ double wave_scan_f64_dpp(double v) {
    v += dpp_fetch_f64<0x111, 0xf>(v);
    v += dpp_fetch_f64<0x112, 0xf>(v);
    v += dpp_fetch_f64<0x114, 0xf>(v);
    v += dpp_fetch_f64<0x118, 0xf>(v);
    v += dpp_fetch_f64<0x142, 0xa>(v);
    v += dpp_fetch_f64<0x143, 0xc>(v);
    return v;
}

/* Each lane asks for `cnt` consecutive places in a list whose length lives in LDS; one atomic
 * per wavefront. Returns the lane's first place. All 64 lanes must call. */
__device__ __forceinline__ int wave_reserve(int cnt, int *counter) {
    const int incl  = wave_scan_i32_dpp(cnt);
    const int total = __shfl(incl, WAVE - 1, WAVE);
    int       base  = 0;
    if ((threadIdx.x & (WAVE - 1)) == WAVE - 1 && total)
        base = atomicAdd(counter, total);
    base = __shfl(base, WAVE - 1, WAVE);
    return base + incl - cnt;
}

/* ---- workgroup combines through LDS -------------------------------------------------------- */
/* Combining without a barrier: every wavefront of the workgroup deposits its part in LDS and
 * then calls this; the call returns true (in all lanes) in the wavefront that arrives last,
 * which finds every part deposited -- the LDS operations of a workgroup are performed in the
 * order they were issued. The others go on without waiting. `counter` (LDS) must hold zero, and
 * a barrier must have published that, before the first arrival. */
__device__ __forceinline__ bool wave_arrives_last(uint32_t *counter) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    uint32_t ticket = 0;
    if ((threadIdx.x & (WAVE - 1)) == 0)
        ticket = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED,
                                        __HIP_MEMORY_SCOPE_WORKGROUP);
    ticket = readlane_u32(ticket, 0);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    return ticket == NWAVES - 1;
}
/* All 256 threads call; every thread receives the maximum. `scratch` holds NWAVES entries. */
__device__ __forceinline__ uint64_t block_max_u64(uint64_t v, uint64_t *scratch) {
    v = wave_max_u64(v);
    if ((threadIdx.x & (WAVE - 1)) == 0)
        scratch[threadIdx.x / WAVE] = v;
    __syncthreads();
    uint64_t r = scratch[0];
#pragma unroll
    for (int w = 1; w < NWAVES; ++w)
        r = scratch[w] > r ? scratch[w] : r;
    __syncthreads();
    return r;
}
/* Sum over the workgroup in a fixed order (lanes by butterfly, then waves 0..3). */
__device__ __forceinline__ double block_sum_f64(double v, double *scratch) {
    v = wave_sum_f64(v);
    if ((threadIdx.x & (WAVE - 1)) == 0)
        scratch[threadIdx.x / WAVE] = v;
    __syncthreads();
    double r = scratch[0];
#pragma unroll
    for (int w = 1; w < NWAVES; ++w)
        r += scratch[w];
    __syncthreads();
    return r;
}
/* NV sums over the workgroup at once (wavefront totals by DPP steps, then the four waves in
 * order): every thread receives all NV totals. `scratch` holds NWAVES * NV entries. */
template <int NV>
__device__ __forceinline__ void block_sum_f64_multi(double (&v)[NV], double *scratch) {
    const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const double t = wave_scan_f64_dpp(v[j]); /* lane 63 holds the wavefront's total */
        if (lane == WAVE - 1)
            scratch[w * NV + j] = t;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        double r = scratch[j];
#pragma unroll
        for (int x = 1; x < NWAVES; ++x)
            r += scratch[x * NV + j];
        v[j] = r;
    }
    __syncthreads();
}
/* Inclusive prefix sum over the 256 threads in thread order; *total receives the sum. */
__device__ __forceinline__ double block_scan_f64(double v, double *scratch, double *total) {
    const int w    = threadIdx.x / WAVE;
    const int lane = threadIdx.x & (WAVE - 1);
    v              = wave_scan_f64(v);
    if (lane == WAVE - 1)
        scratch[w] = v;
    __syncthreads();
    double off = 0.0, all = 0.0;
#pragma unroll
    for (int i = 0; i < NWAVES; ++i) {
        if (i < w)
            off += scratch[i];
        all += scratch[i];
    }
    __syncthreads();
    if (total)
        *total = all;
    return v + off;
}
__device__ __forceinline__ int block_scan_i32(int v, int *scratch, int *total) {
    const int w    = threadIdx.x / WAVE;
    const int lane = threadIdx.x & (WAVE - 1);
    v              = wave_scan_i32(v);
    if (lane == WAVE - 1)
        scratch[w] = v;
    __syncthreads();
    int off = 0, all = 0;
#pragma unroll
    for (int i = 0; i < NWAVES; ++i) {
        if (i < w)
            off += scratch[i];
        all += scratch[i];
    }
    __syncthreads();
    if (total)
        *total = all;
    return v + off;
}

/* ---- the logit transform applied while a chunk is read ------------------------------------ */

/* Penalty arithmetic; every step rounds once, matching the CPU statement of the same rule.
 * l / rep is formed as (float)((double)l * inv_rep), inv_rep = 1.0 / (double)rep rounded once on
 * the host: the product is within 2^-51 of the quotient while the quotient of two binary32
 * values stays at least 2^-49 (relative) away from every midpoint between neighbouring binary32
 * values, so the single rounding to binary32 lands where the division's would. It replaces a
 * twelve-instruction division sequence by three instructions. Tiny and non-finite values divide. */
__device__ __forceinline__ float penalise(float l, uint32_t count, float rep, double inv_rep,
                                          float freq, float pres) {
    if (l > 0.0f) {
        if (__builtin_expect(l >= 0x1p-60f && l <= 0x1p60f && rep >= 0x1p-20f && rep <= 0x1p20f, 1))
            l = (float) ((double) l * inv_rep);
        else
            l = __fdiv_rn(l, rep);
    } else {
        l = __fmul_rn(l, rep);
    }
    l = __fsub_rn(l, __fmul_rn(freq, (float) count));
    l = __fsub_rn(l, pres);
    return l;
}

/* The history lookup of one chunk, in two steps so that the logit loads can be in flight while
 * the history is read: history_clear() zeroes the table (ends with a barrier), history_count()
 * adds the occurrences of each vocabulary id of [base, end) in the row's history (ends with a
 * barrier). cnt16 packs two 16-bit counters per word: histories are capped at 65535 entries.
 * Ids outside the row's vocabulary fall outside every chunk and are ignored. */
template <int CHUNK>
__device__ __forceinline__ void history_clear(uint32_t *cnt16) {
    uint4 *p = reinterpret_cast<uint4 *>(cnt16);
    for (int i = threadIdx.x; i < CHUNK / 8; i += TPB)
        p[i] = make_uint4(0u, 0u, 0u, 0u);
    lds_barrier();
}
/* Reading a row's history in two steps so that its loads are in flight early:
 * history_prefetch() issues the loads of the row's length and of the first 8 ids per thread
 * (4 ids per load; an unaligned history is read id by id later), history_for_each() then
 * calls f(id) for every entry, the workgroup's threads sharing the entries. */
struct HistPrefetch {
    int4 a, b;
    int  len;
    bool vec;
};
/* `n_rows` is the number of rows of the launch. The row's length is fetched with a vector load
 * (each lane reads the length of a following row, lane 0 its own): a scalar load here would
 * sit in the same counter as the LDS traffic and stall the first barrier until it returns. */
__device__ __forceinline__ HistPrefetch history_prefetch(const RowView &rv, int row, int n_rows) {
    HistPrefetch   pf;
    const int32_t *h   = rv.hist + (long) row * rv.hist_ld;
    const int      ld4 = (int) (rv.hist_ld >> 2);
    const int      g   = threadIdx.x;
    {
        int r = row + (int) (threadIdx.x & (WAVE - 1));
        r     = r < n_rows ? r : n_rows - 1;
        pf.len = rv.hist_len[r]; /* lane 0 holds this row's length; broadcast when consumed */
    }
    pf.vec             = (((uintptr_t) h) & 15) == 0;
    const int4 *h4     = reinterpret_cast<const int4 *>(h);
    pf.a               = make_int4(-1, -1, -1, -1);
    pf.b               = make_int4(-1, -1, -1, -1);
    if (pf.vec && g < ld4)
        pf.a = h4[g];
    if (pf.vec && g + TPB < ld4)
        pf.b = h4[g + TPB];
    return pf;
}
template <typename F>
__device__ __forceinline__ void history_for_each(const RowView &rv, int row,
                                                 const HistPrefetch &pf, F &&f) {
    int len = __builtin_amdgcn_readfirstlane(pf.len);
    if (len > rv.hist_ld)
        len = (int) rv.hist_ld;
    const int32_t *h  = rv.hist + (long) row * rv.hist_ld;
    int            i0 = 0;
    if (pf.vec) {
        const int4 *h4 = reinterpret_cast<const int4 *>(h);
        const int   n4 = len >> 2;
        const int   g  = threadIdx.x;
        if (g < n4) {
            f(pf.a.x);
            f(pf.a.y);
            f(pf.a.z);
            f(pf.a.w);
        }
        if (g + TPB < n4) {
            f(pf.b.x);
            f(pf.b.y);
            f(pf.b.z);
            f(pf.b.w);
        }
        for (int g2 = g + 2 * TPB; g2 < n4; g2 += 2 * TPB) {
            const int4 a = h4[g2];
            const int4 b = g2 + TPB < n4 ? h4[g2 + TPB] : make_int4(-1, -1, -1, -1);
            f(a.x);
            f(a.y);
            f(a.z);
            f(a.w);
            f(b.x);
            f(b.y);
            f(b.z);
            f(b.w);
        }
        i0 = n4 << 2;
    }
    for (int i = i0 + threadIdx.x; i < len; i += TPB)
        f(h[i]);
}
/* Two-phase variant for lookups that go through LDS: look(id) is evaluated for up to eight
 * entries before apply(code) runs for each of them, so the eight LDS reads are in flight together
 * instead of each waiting behind the previous entry's atomic. */
template <typename L, typename A>
__device__ __forceinline__ void history_for_each_batched(const RowView &rv, int row,
                                                         const HistPrefetch &pf, L &&look,
                                                         A &&apply) {
    int len = __builtin_amdgcn_readfirstlane(pf.len);
    if (len > rv.hist_ld)
        len = (int) rv.hist_ld;
    const int32_t *h  = rv.hist + (long) row * rv.hist_ld;
    int            i0 = 0;
    auto           eight = [&](const int4 &a, const int4 &b) {
        const int c0 = look(a.x), c1 = look(a.y), c2 = look(a.z), c3 = look(a.w);
        const int c4 = look(b.x), c5 = look(b.y), c6 = look(b.z), c7 = look(b.w);
        apply(c0);
        apply(c1);
        apply(c2);
        apply(c3);
        apply(c4);
        apply(c5);
        apply(c6);
        apply(c7);
    };
    if (pf.vec) {
        const int4 *h4   = reinterpret_cast<const int4 *>(h);
        const int   n4   = len >> 2;
        const int   g    = threadIdx.x;
        const int4  none = make_int4(-1, -1, -1, -1);
        if (g < n4)
            eight(pf.a, g + TPB < n4 ? pf.b : none);
        for (int g2 = g + 2 * TPB; g2 < n4; g2 += 2 * TPB)
            eight(h4[g2], g2 + TPB < n4 ? h4[g2 + TPB] : none);
        i0 = n4 << 2;
    }
    for (int i = i0 + threadIdx.x; i < len; i += TPB)
        apply(look(h[i]));
}
__device__ __forceinline__ void history_count(const RowView &rv, int row, const HistPrefetch &pf,
                                              int base, int end, uint32_t *cnt16) {
    history_for_each(rv, row, pf, [&](int t) {
        const int off = t - base;
        if (off >= 0 && t < end)
            atomicAdd(&cnt16[off >> 1], 1u << (16 * (off & 1)));
    });
    lds_barrier();
}

/* A 16-byte load marked non-temporal: the line is not kept in the caches on its way. For rows
 * that come from HBM and are read once this is the faster read (a launch over 32.8 MB: 6.4 us
 * against 7.0 us); for rows still in the Infinity Cache it is the slower one (5.5 us against
 * 3.4 us), so it is used only where the caller has said the logits are not cache-resident. */
__device__ __forceinline__ float4 load_streaming(const float4 *p) {
    typedef float nt_f4 __attribute__((ext_vector_type(4)));
    const nt_f4 t = __builtin_nontemporal_load(reinterpret_cast<const nt_f4 *>(p));
    return make_float4(t.x, t.y, t.z, t.w);
}

/* Issues the loads of the chunk [base, end) of a row into registers (layout in the file
 * header). Positions at or beyond `end` hold -inf. */
template <int NV>
__device__ __forceinline__ void load_raw(const RowView &rv, const float *__restrict__ row,
                                         int base, int end, float4 (&v)[NV],
                                         int tid = (int) threadIdx.x) {
    const float ninf = -__builtin_inff();
    if (rv.vec_ok && end - base == NV * TPB * 4) { /* full chunk: no per-element tests */
        const float4 *p = reinterpret_cast<const float4 *>(row + base) + tid;
        if (rv.stream_loads) {
#pragma unroll
            for (int j = 0; j < NV; ++j)
                v[j] = load_streaming(p + j * TPB);
        } else {
#pragma unroll
            for (int j = 0; j < NV; ++j)
                v[j] = p[j * TPB];
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int e = base + 4 * (j * TPB + tid);
        if (rv.vec_ok && e + 3 < end) {
            v[j] = *reinterpret_cast<const float4 *>(row + e);
        } else {
            v[j].x = e + 0 < end ? row[e + 0] : ninf;
            v[j].y = e + 1 < end ? row[e + 1] : ninf;
            v[j].z = e + 2 < end ? row[e + 2] : ninf;
            v[j].w = e + 3 < end ? row[e + 3] : ninf;
        }
    }
}

/* Allowed-token mask: the four mask bits of elements e .. e + 3 of a row (e a multiple of 4,
 * below n_vocab), bit c set = element e + c may be sampled. Only called with rv.allowed set. */
__device__ __forceinline__ uint32_t allowed_nibble(const RowView &rv, long row, int e) {
    const uint32_t *m = rv.allowed + row * rv.allowed_ld;
    return (m[e >> 5] >> (e & 31)) & 0xfu;
}
__device__ __forceinline__ bool allowed_at(const RowView &rv, long row, int e) {
    const uint32_t *m = rv.allowed + row * rv.allowed_ld;
    return (m[e >> 5] >> (e & 31)) & 1u;
}

/* The logit soft-cap, tanhf(x / cap) * cap (head.c:148-159), kept out of line: few models have
 * one, and glibc's tanhf is some two hundred instructions per element -- inlined at every site
 * it would multiply the size of every kernel and evict the code that does run from the
 * instruction cache. Arguments and results travel in registers. */
__device__ __noinline__ float softcap1(float x, float cap) {
    return __fmul_rn(geist_tanhf_glibc(__fdiv_rn(x, cap)), cap);
}
__device__ __noinline__ float4 softcap4(float4 v, float cap) {
    v.x = __fmul_rn(geist_tanhf_glibc(__fdiv_rn(v.x, cap)), cap);
    v.y = __fmul_rn(geist_tanhf_glibc(__fdiv_rn(v.y, cap)), cap);
    v.z = __fmul_rn(geist_tanhf_glibc(__fdiv_rn(v.z, cap)), cap);
    v.w = __fmul_rn(geist_tanhf_glibc(__fdiv_rn(v.w, cap)), cap);
    return v;
}

/* Penalties (when cnt16 != NULL) and the soft-cap on a chunk held in registers. */
template <int NV>
__device__ __forceinline__ void apply_transform(const RowView &rv, const uint32_t *cnt16,
                                                float4 (&v)[NV]) {
    const int tid = threadIdx.x;
    if (cnt16) {
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int   off = 4 * (j * TPB + tid); /* even, so two words cover the float4 */
            const uint2 w   = *reinterpret_cast<const uint2 *>(cnt16 + (off >> 1));
            if (w.x | w.y) {
                if (w.x & 0xffffu)
                    v[j].x = penalise(v[j].x, w.x & 0xffffu, rv.rep, rv.inv_rep, rv.freq, rv.pres);
                if (w.x >> 16)
                    v[j].y = penalise(v[j].y, w.x >> 16, rv.rep, rv.inv_rep, rv.freq, rv.pres);
                if (w.y & 0xffffu)
                    v[j].z = penalise(v[j].z, w.y & 0xffffu, rv.rep, rv.inv_rep, rv.freq, rv.pres);
                if (w.y >> 16)
                    v[j].w = penalise(v[j].w, w.y >> 16, rv.rep, rv.inv_rep, rv.freq, rv.pres);
            }
        }
    }
    if (rv.softcap > 0.0f) {
        const float c = rv.softcap;
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            v[j] = softcap4(v[j], c);
        }
    }
}

/* The transforms of one float4 group of a chunk in registers -- elements base + off .. + 3,
 * off = 4 * (j * TPB + tid) -- for kernels that work through a chunk group by group while the
 * later groups' loads are still in flight: penalties from the count table, soft-cap, chunk
 * padding back to -inf, allowed-token mask. The same values as fetch_chunk() produces. */
template <bool PEN, bool EXTRAS = true>
__device__ __forceinline__ void transform_group(const RowView &rv, long row, const uint32_t *cnt16,
                                                int off, int base, int end, float4 &q) {
    if (PEN) {
        const uint2 w = *reinterpret_cast<const uint2 *>(cnt16 + (off >> 1));
        if (w.x | w.y) {
            if (w.x & 0xffffu)
                q.x = penalise(q.x, w.x & 0xffffu, rv.rep, rv.inv_rep, rv.freq, rv.pres);
            if (w.x >> 16)
                q.y = penalise(q.y, w.x >> 16, rv.rep, rv.inv_rep, rv.freq, rv.pres);
            if (w.y & 0xffffu)
                q.z = penalise(q.z, w.y & 0xffffu, rv.rep, rv.inv_rep, rv.freq, rv.pres);
            if (w.y >> 16)
                q.w = penalise(q.w, w.y >> 16, rv.rep, rv.inv_rep, rv.freq, rv.pres);
        }
    }
    if (!EXTRAS) /* the caller knows: no soft-cap, no padding, no mask */
        return;
    if (rv.softcap > 0.0f) {
        q           = softcap4(q, rv.softcap);
        const int l = end - base - off; /* elements of the group inside the row */
        q.x         = l > 0 ? q.x : -__builtin_inff();
        q.y         = l > 1 ? q.y : -__builtin_inff();
        q.z         = l > 2 ? q.z : -__builtin_inff();
        q.w         = l > 3 ? q.w : -__builtin_inff();
    }
    if (rv.allowed && base + off < end) {
        const uint32_t ok = allowed_nibble(rv, row, base + off);
        q.x               = (ok & 1u) ? q.x : -__builtin_inff();
        q.y               = (ok & 2u) ? q.y : -__builtin_inff();
        q.z               = (ok & 4u) ? q.z : -__builtin_inff();
        q.w               = (ok & 8u) ? q.w : -__builtin_inff();
    }
}

/* max of three floats in one instruction. Unlike fmaxf() no canonicalising self-max is emitted
 * per operand; a quiet NaN operand is ignored (a signalling NaN may come back quieted, which
 * only makes the caller keep more candidates). */
__device__ __forceinline__ float max3f(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ float f4_max(const float4 &q) { return max3f(max3f(q.x, q.y, q.z), q.w, q.w); }

__device__ __forceinline__ float f4_get(const float4 &q, int c) {
    return c == 0 ? q.x : c == 1 ? q.y : c == 2 ? q.z : q.w;
}

/* fp32 steps of the reference's softmax argument, (l - max) * inv_t (sampler.c:80), kept as
 * two separately rounded operations. */
__device__ __forceinline__ float softmax_arg(float l, float mx, float inv_t) {
    return __fmul_rn(__fsub_rn(l, mx), inv_t);
}

/* z bin of an element: z = -(softmax argument) >= 0 in steps of 1/ZBIN_PER_NAT, truncated;
 * -inf and everything past the last bin land in ZBINS - 1 or above (callers clamp or skip). The
 * exp-sum pass and the candidate pass must agree on it bit for bit, hence one function. */
__device__ __forceinline__ int zbin(float arg) {
    const float z = __fmul_rn(arg, -(float) ZBIN_PER_NAT);
    return z < (float) (ZBINS - 1) ? (int) z : ZBINS - 1;
}

/* zbin(arg) <= b, as one comparison: the scaling in zbin() is by a power of two, hence exact,
 * and truncation keeps z < b + 1, so the test is arg > -(b + 1) / ZBIN_PER_NAT (false for NaN,
 * as zbin's last bin is). */
__device__ __forceinline__ float zbin_threshold(int b) {
    return -(float) (b + 1) / (float) ZBIN_PER_NAT;
}

} // namespace gs
#endif
