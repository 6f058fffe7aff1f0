/*
 * sampler_walk.h -- the index-order walk the temperature sampler (src/engine/sampler.c:90-102),
 * the bonus token and the residual resampling of speculative verification share. Included by
 * sampler_kernels.hip.
 *
 * A row is never walked from its start. The streaming pass leaves, per chunk, the sum of the
 * weights and the sums of the chunk's slabs: slab j of a chunk is the 1024 consecutive elements
 * the threads t = 0..255 hold as their j-th float4, positions base + 4 * (j * 256 + t) + c.
 * Index order inside a chunk is (slab, thread, component), so the chunk is located from the chunk
 * sums, the slab from the slab sums, and only that slab is read again: 4 elements per thread,
 * one workgroup scan.
 */
#ifndef GEIST_SAMPLER_WALK_H
#define GEIST_SAMPLER_WALK_H

namespace gs {


/* The four weights thread `tid` owns in a slab: p_i (temperature walk) or max(0, pn_i - q_i)
 * (residual walk). Positions at or beyond `end` weigh 0. */
template <bool RESID>
__device__ __forceinline__ void slab_weights(const float4 &v, const float4 &qv, int e, int end,
                                             float mx, float inv_t, double sum,
                                             const uint64_t *tab, float (&w)[4]) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        float x = 0.0f;
        if (e + c < end) {
            const float p = geist_expf_glibc_le0(softmax_arg(f4_get(v, c), mx, inv_t), tab);
            if (RESID) {
                const float r = __fsub_rn((float) ((double) p / sum), f4_get(qv, c));
                x             = r > 0.0f ? r : 0.0f;
            } else {
                x = p;
            }
        }
        w[c] = x;
    }
}

/* Draft probabilities of a chunk. qrow == NULL: the drafter proposed its token with certainty
 * (an n-gram lookup, src/engine/session.c:437-513), q is 1 at `x` and 0 elsewhere. */
template <int NV>
__device__ __forceinline__ void load_q_chunk(const float *qrow, bool vec, int x, int base, int end,
                                             float4 (&qv)[NV]) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int e = base + 4 * (j * TPB + tid);
        if (qrow == nullptr) {
            qv[j].x = e + 0 == x ? 1.f : 0.f;
            qv[j].y = e + 1 == x ? 1.f : 0.f;
            qv[j].z = e + 2 == x ? 1.f : 0.f;
            qv[j].w = e + 3 == x ? 1.f : 0.f;
        } else if (vec && e + 3 < end) {
            qv[j] = *reinterpret_cast<const float4 *>(qrow + e);
        } else {
            qv[j].x = e + 0 < end ? qrow[e + 0] : 0.f;
            qv[j].y = e + 1 < end ? qrow[e + 1] : 0.f;
            qv[j].z = e + 2 < end ? qrow[e + 2] : 0.f;
            qv[j].w = e + 3 < end ? qrow[e + 3] : 0.f;
        }
    }
}

struct WalkShared {
    double scan[NWAVES];
    double before, target;
    int    chunk, slab, pick, last_pos;
};

/* First step of the walk, by the first wavefront (all its lanes call): the chunk in which the
 * running sum of chunk_w (C weights in LDS) first exceeds u * (their sum), C - 1 if none does.
 * Lane l holds chunks l and l + 64 (MAX_CHUNKS = 128), the running sums come from DPP scans, the
 * first chunk past the target from a ballot. Returns the chunk; *run receives the running sum
 * before it, *target the target (the same in every lane). */
__device__ __forceinline__ int walk_locate_chunk(const double *chunk_w, int C, float u, double *run,
                                                 double *target) {
    static_assert(MAX_CHUNKS <= 2 * WAVE, "two chunks per lane");
    const int    lane = threadIdx.x & (WAVE - 1);
    const double w0   = lane < C ? chunk_w[lane] : 0.0;
    const double w1   = lane + WAVE < C ? chunk_w[lane + WAVE] : 0.0;
    const double i0   = wave_scan_f64_dpp(w0);
    const double h0   = __shfl(i0, WAVE - 1, WAVE);
    const double i1   = h0 + wave_scan_f64_dpp(w1);
    const double tot  = __shfl(i1, WAVE - 1, WAVE);
    *target           = (double) u * tot;
    const uint64_t b0 = __ballot(lane < C && *target < i0);
    const uint64_t b1 = __ballot(lane + WAVE < C && *target < i1);
    int            at = C - 1;
    if (b0)
        at = __ffsll((long long) b0) - 1;
    else if (b1)
        at = WAVE + __ffsll((long long) b1) - 1;
    /* running sum before chunk `at`: the inclusive sum of the lane before it */
    const double p0 = __shfl_up(i0, 1, WAVE), p1 = __shfl_up(i1, 1, WAVE);
    const double e0 = lane ? p0 : 0.0, e1 = lane ? p1 : h0;
    *run            = at < WAVE ? __shfl(e0, at, WAVE) : __shfl(e1, at - WAVE, WAVE);
    return at;
}
/* Second step, same wavefront: the slab of the located chunk, from the chunk's NV slab weights
 * (`slab_w`, LDS or global memory; lane j holds slab j). *run comes in as the running sum before
 * the chunk and leaves as the running sum before the slab. */
template <int NV>
__device__ __forceinline__ int walk_locate_slab(const double *slab_w, double target, double *run) {
    const int      lane = threadIdx.x & (WAVE - 1);
    const double   sw   = lane < NV ? slab_w[lane] : 0.0;
    const double   si   = *run + wave_scan_f64_dpp(sw);
    const uint64_t bs   = __ballot(lane < NV && target < si);
    const int      js   = bs ? __ffsll((long long) bs) - 1 : NV - 1;
    const double   ps   = __shfl_up(si, 1, WAVE);
    *run                = __shfl(lane ? ps : *run, js, WAVE);
    return js;
}

/* One slab's step of the walk, by the whole workgroup: thread `tid` brings the slab's four
 * weights it owns (elements e .. e + 3, `send` the end of the slab), `carry` is the running sum
 * before the slab. Returns true once an element has been picked (sh.pick); otherwise `carry` has
 * moved past the slab. */
template <bool RESID>
__device__ __forceinline__ bool walk_slab_step(const float (&w)[4], int e, int send, double target,
                                               double &carry, WalkShared &sh) {
    const double part = (double) w[0] + (double) w[1] + (double) w[2] + (double) w[3];
    double       slab;
    const double incl = block_scan_f64(part, sh.scan, &slab);
    double       run  = carry + (incl - part);
    int          lastpos = -1;
    uint32_t     pick    = 0x7fffffffu;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        run += (double) w[c];
        if (w[c] > 0.0f)
            lastpos = e + c;
        if (pick == 0x7fffffffu && e + c < send && w[c] > 0.0f && target < run)
            pick = (uint32_t) (e + c); /* the thread's first: the running sum only grows */
    }
    /* one atomic per wavefront: nearly every thread has a last position to report, and 256
     * atomics on one word of LDS took 4 us */
    pick = ~wave_max_u32(~pick);
    if (RESID)
        lastpos = (int) wave_max_u32((uint32_t) (lastpos + 1)) - 1;
    if ((threadIdx.x & (WAVE - 1)) == 0) {
        if (pick != 0x7fffffffu)
            atomicMin(&sh.pick, (int) pick);
        if (RESID && lastpos >= 0)
            atomicMax(&sh.last_pos, lastpos);
    }
    __syncthreads();
    if (sh.pick != 0x7fffffff)
        return true;
    carry += slab;
    __syncthreads();
    return false;
}

/* The walk from slab `slab0` of chunk `chunk0` on, reading the row: slab after slab, chunk after
 * chunk, until an element is picked or the row ends. sh.pick / sh.last_pos carry the result;
 * `end_out` receives the end of the last chunk looked at. */
template <int NV, bool PEN, bool RESID>
__device__ __forceinline__ void walk_from(const RowView &rv, int row, int n_rows, int C, int chunk0,
                                          int slab0, double carry, double target, float mx,
                                          float inv_t, double sum, const float *qrow, bool qvec,
                                          int qx, const uint64_t *tab, uint32_t *s_cnt16,
                                          WalkShared &sh, int &end_out) {
    const int tid = threadIdx.x;
    int       base, end = end_out;
    bool      found = false;
    for (int chunk = chunk0; chunk < C && !found; ++chunk) {
        chunk_bounds<NV>(rv, chunk, base, end);
        for (int j = chunk == chunk0 ? slab0 : 0; j < NV; ++j) {
            const int sbase = base + j * 4 * TPB;
            if (sbase >= end)
                break;
            const int send = sbase + 4 * TPB < end ? sbase + 4 * TPB : end;
            float4    v[1], qv[1];
            /* a slab is a chunk of 1024 */
            fetch_chunk<1, PEN>(rv, row, n_rows, sbase, send, s_cnt16, v);
            qv[0] = v[0];
            if (RESID)
                load_q_chunk<1>(qrow, qvec, qx, sbase, send, qv);
            const int e = sbase + 4 * tid;
            float     w[4];
            slab_weights<RESID>(v[0], qv[0], e, send, mx, inv_t, sum, tab, w);
            if (walk_slab_step<RESID>(w, e, send, target, carry, sh)) {
                found = true;
                break;
            }
        }
    }
    end_out = end;
}

/* Walks row `row` in index order for the first element at which the running weight exceeds
 * u * (sum of chunk_w). chunk_w: C per-chunk weights in LDS; slab_w: the row's C * SLABS_MAX slab
 * weights in global memory, or NULL where the pass did not keep them (the located chunk is then
 * walked from its first slab); NV: slabs per chunk of the pass that wrote them; qrow / qx: the
 * draft probabilities of the residual walk (see load_q_chunk). Returns the id to
 * every thread. Should rounding leave the target beyond the located slab, the walk goes on through
 * the following slabs and chunks, as the reference's single loop does (sampler.c:93-99); past the
 * end of the row it returns the row's last index (sampler.c:100-101), for the residual walk the
 * last element seen with a positive weight. */
template <int NV, bool PEN, bool RESID>
__device__ int index_order_walk(const RowView &rv, int row, int n_rows, const double *chunk_w,
                                const double *__restrict__ slab_w, int C, float u, float mx,
                                float inv_t, double sum, const float *qrow, bool qvec, int qx,
                                const uint64_t *tab, uint32_t *s_cnt16, WalkShared &sh) {
    const int tid = threadIdx.x;
    if (tid < WAVE) {
        double    run, target;
        const int at = walk_locate_chunk(chunk_w, C, u, &run, &target);
        /* without slab weights the located chunk is walked from its first slab */
        const int js = slab_w ? walk_locate_slab<NV>(slab_w + at * SLABS_MAX, target, &run) : 0;
        if (tid == 0) {
            sh.chunk    = at;
            sh.slab     = js;
            sh.before   = run;
            sh.target   = target;
            sh.pick     = 0x7fffffff;
            sh.last_pos = -1;
        }
    }
    __syncthreads();
    int end = 0;
    walk_from<NV, PEN, RESID>(rv, row, n_rows, C, sh.chunk, sh.slab, sh.before, sh.target, mx, inv_t,
                              sum, qrow, qvec, qx, tab, s_cnt16, sh, end);
    __syncthreads();
    int tok = sh.pick;
    if (tok == 0x7fffffff)
        tok = RESID && sh.last_pos >= 0 ? sh.last_pos : end - 1;
    __syncthreads();
    return tok;
}

} // namespace gs
#endif
