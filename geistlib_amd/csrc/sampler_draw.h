/*
 * sampler_draw.h -- the temperature draw (src/engine/sampler.c:68-102) in ONE kernel. Included by
 * sampler_kernels.hip.
 *
 * k_scan_expsum followed by k_final_temperature reads the row once, but the second kernel reads
 * one slab of it again and costs a launch; for a single row that launch is half the step. Here
 * the workgroups of a row meet twice: once for the row's maximum (row_best_meet), once more
 * for the chunks' sums (row_sums_meet). Every workgroup then knows all chunk sums, works out in
 * which chunk the draw u * sum falls -- the same arithmetic on the same numbers in each of them,
 * so exactly one finds the draw in its own chunk -- and that one walks its chunk from the
 * registers it still holds. Results are those of the two-kernel form bit for bit: the sums are
 * formed in the same order (chunk_slab_totals), the walk is the same code (sampler_walk.h).
 *
 * The waits are bounded like the first meet's. A workgroup that gives up a wait forms what it
 * is missing itself, from the row: the maximum as before, the other chunks' sums by running
 * the same summation over each of them (all workgroups that do so get the same bits, so they
 * still agree on the chunk), and then, if the draw is its own, walks from memory. Every
 * workgroup ends whatever the others do.
 */
#ifndef GEIST_SAMPLER_DRAW_H
#define GEIST_SAMPLER_DRAW_H

namespace gs {

/* A wavefront's share of a chunk's slab sums: sum j over the lanes of Σ_c expf(arg) of group j,
 * into s_sum[w * NV + j]. NV == 8 goes through the wavefront's 8 x 64 table `tr` in LDS (see
 * expsum_chunk), NV == 2 through two DPP scans: the same operations in the same order as the
 * SLABS form of expsum_chunk. On return v[] holds the weights themselves (expf of each element's
 * argument; 0 at positions beyond the row, which were -inf) in place of the logits. */
template <int NV>
__device__ __forceinline__ void chunk_slab_totals(float4 (&v)[NV], float mx, float inv_t,
                                                  const uint64_t *s_tab, double *s_tr,
                                                  double *s_sum) {
    const int        tid = threadIdx.x, lane = tid & (WAVE - 1), w = tid / WAVE;
    constexpr bool   TRANSPOSED = NV == 8;
    volatile double *tr = s_tr + w * (8 * WAVE);
    double           accs[TRANSPOSED ? 1 : NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        double a4;
        float  pw[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            pw[c]          = geist_expf_glibc_le0(softmax_arg(f4_get(v[j], c), mx, inv_t), s_tab);
            const double p = (double) pw[c];
            a4 = c == 0 ? p : a4 + p;
        }
        v[j] = make_float4(pw[0], pw[1], pw[2], pw[3]); /* kept for the walk */
        if (TRANSPOSED)
            tr[j * WAVE + (lane ^ j)] = a4;
        else
            accs[j] = a4;
        if (j + 1 < NV) { /* one group at a time, see expsum_chunk */
            if (TRANSPOSED)
                asm volatile("" : "+v"(a4), "+v"(v[j + 1].x), "+v"(v[j + 1].y), "+v"(v[j + 1].z),
                                  "+v"(v[j + 1].w));
            else
                asm volatile("" : "+v"(accs[j]), "+v"(v[j + 1].x), "+v"(v[j + 1].y),
                                  "+v"(v[j + 1].z), "+v"(v[j + 1].w));
        }
    }
    if (TRANSPOSED) {
        const int g = lane >> 3, first = 8 * (lane & 7);
        double    r = tr[g * WAVE + (first ^ g)];
#pragma unroll
        for (int i = 1; i < 8; ++i)
            r += tr[g * WAVE + ((first + i) ^ g)];
        r += dpp_fetch_f64<0x111, 0xf>(r);
        r += dpp_fetch_f64<0x112, 0xf>(r);
        r += dpp_fetch_f64<0x114, 0xf>(r);
        if ((lane & 7) == 7)
            s_sum[w * NV + g] = r;
    } else {
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const double t = wave_scan_f64_dpp(accs[j]);
            if (lane == WAVE - 1)
                s_sum[w * NV + j] = t;
        }
    }
}
/* by one lane, once all four wavefronts have deposited: the chunk's slab sums (wavefront 0..3
 * in order) into slab[], their sum in slab order returned */
template <int NV>
__device__ __forceinline__ double combine_slab_totals(const double *s_sum, double *slab) {
    double total = 0.0;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        double r = s_sum[j];
#pragma unroll
        for (int x = 1; x < NWAVES; ++x)
            r += s_sum[x * NV + j];
        slab[j] = r;
        total += r;
    }
    return total;
}

struct DrawShared {
    double     slab[SLABS_MAX]; /* this chunk's slab sums */
    double     csum[MAX_CHUNKS];
    double     total;
    int        have_sums;
    WalkShared walk;
};

/* The second meet: the reporting wavefront stores its chunk's sum into the chunk's slot (bits
 * + 1, never zero: sums are finite and not negative, or NaN patterns short of all ones) and
 * polls the row's slots like row_best_meet; met, it leaves every chunk's sum in sh.csum and
 * sh.have_sums = 1. Not met (or `wait` false: the first meet already gave up, the others may
 * not even have started): sh.have_sums = 0. Ends with a barrier. */
__device__ __forceinline__ void row_sums_meet(uint64_t *row_slots, int chunk, int C, double total,
                                              bool reporter, bool wait, uint32_t wait_limit,
                                              DrawShared &sh, uint32_t local = 0) {
    const int lane = threadIdx.x & (WAVE - 1);
    if (reporter) {
        if (lane == 0)
            meet_store(row_slots + chunk, (uint64_t) __double_as_longlong(total) + 1u, local);
        uint64_t a = 0, b = 0;
        uint32_t polls = 0;
        bool     met   = wait;
        while (met) {
            a = lane < C ? __hip_atomic_load(row_slots + lane, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT)
                         : 1;
            b = lane + WAVE < C ? __hip_atomic_load(row_slots + lane + WAVE, __ATOMIC_RELAXED,
                                                    __HIP_MEMORY_SCOPE_AGENT)
                                : 1;
            if (__builtin_amdgcn_ballot_w64(a == 0 || b == 0) == 0)
                break;
            if (++polls > wait_limit)
                met = false;
        }
        if (met) {
            if (lane < C)
                sh.csum[lane] = __longlong_as_double((long long) (a - 1u));
            if (lane + WAVE < C)
                sh.csum[lane + WAVE] = __longlong_as_double((long long) (b - 1u));
        }
        if (lane == 0)
            sh.have_sums = met ? 1 : 0;
    }
    __syncthreads();
}

template <int NV, bool PEN, bool PLAIN>
__device__ __forceinline__ void draw_chunk(const RowView &rv, int row, int chunk, int n_rows,
                                           int base, int end, float inv_t,
                                           const float *__restrict__ uniforms,
                                           int32_t *__restrict__ out, uint64_t *sum_slots,
                                           uint32_t *s_cnt16, double *s_sum, uint64_t *s_tab,
                                           uint64_t tabv, double *s_tr, DrawShared &sh,
                                           const FusedScan &fs) {
    const int tid = threadIdx.x, C = rv.n_chunks;
    if (PEN)
        __builtin_amdgcn_s_setprio(3); /* see expsum_chunk */
    const float u_row = uniforms[row];
    HistPrefetch pf;
    if (PEN)
        pf = history_prefetch(rv, row, n_rows);
    float4       v[NV];
    const float *rowp = rv.logits + (long) row * rv.ld;
    if (PLAIN) {
        const float4 *p = reinterpret_cast<const float4 *>(rowp + base) + tid;
        if (rv.stream_loads) {
#pragma unroll
            for (int j = 0; j < NV; ++j)
                v[j] = load_streaming(p + j * TPB);
        } else {
#pragma unroll
            for (int j = 0; j < NV; ++j)
                v[j] = p[j * TPB];
        }
    } else {
        load_raw<NV>(rv, rowp, base, end, v);
    }
    if (tid < 32)
        s_tab[tid] = tabv;
    if (tid < 2)
        fs.s_arrive[tid] = 0;
    if (PEN) {
        history_clear<NV * TPB * 4>(s_cnt16);
        history_count(rv, row, pf, base, end, s_cnt16);
    } else {
        lds_barrier();
    }
    /* the chunk's maximum and the row's, as in expsum_chunk */
    float tm = -__builtin_inff();
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        transform_group<PEN, !PLAIN>(rv, row, s_cnt16, 4 * (j * TPB + tid), base, end, v[j]);
        tm = max3f(tm, max3f(v[j].x, v[j].y, v[j].z), v[j].w);
    }
    if (base + 4 * tid >= end)
        tm = __builtin_nanf("");
    const uint32_t bk   = wave_max_u32(f2key(tm));
    uint64_t       best = wave_first_of<NV, PLAIN>(v, bk, base, end);
    if ((tid & (WAVE - 1)) == 0)
        fs.s_red[tid / WAVE] = best;
    const bool last = wave_arrives_last(fs.s_arrive);
    if (last) {
        best = fs.s_red[0];
#pragma unroll
        for (int w = 1; w < NWAVES; ++w)
            best = fs.s_red[w] > best ? fs.s_red[w] : best;
        if (!best)
            best = pack_best(0u, (uint32_t) base);
    }
    bool           met_max = true;
    const uint64_t bb =
        row_best_meet<NV, PEN>(rv, row, chunk, n_rows, best, last, fs, s_cnt16, &met_max);
    if (PEN)
        __builtin_amdgcn_s_setprio(0);
    const float mx = key2f(best_key(bb));

    /* the chunk's slab sums; the wavefront that deposits last combines them and meets the
     * row's other chunks for theirs */
    chunk_slab_totals<NV>(v, mx, inv_t, s_tab, s_tr, s_sum);
    const bool last2 = wave_arrives_last(fs.s_arrive + 1);
    if (last2 && (tid & (WAVE - 1)) == 0)
        sh.total = combine_slab_totals<NV>(s_sum, sh.slab);
    /* (the reporter's lane 0 wrote sh.total: its own LDS write, read back in order) */
    row_sums_meet(sum_slots + (long) row * C, chunk, C, last2 ? sh.total : 0.0, last2, met_max,
                  fs.wait_limit, sh, fs.local);
    const bool from_registers = sh.have_sums != 0;
    if (!from_registers) {
        /* not met: every other chunk's sum by this workgroup, with the same summation */
        if (tid == 0)
            sh.csum[chunk] = sh.total;
        for (int c2 = 0; c2 < C; ++c2) {
            if (c2 == chunk)
                continue;
            int b2, e2;
            chunk_bounds<NV>(rv, c2, b2, e2);
            __syncthreads(); /* the count table and the table of the sums share their memory */
            fetch_chunk<NV, PEN>(rv, row, n_rows, b2, e2, s_cnt16, v);
            __syncthreads();
            double slab2[SLABS_MAX];
            chunk_slab_totals<NV>(v, mx, inv_t, s_tab, s_tr, s_sum);
            __syncthreads();
            if (tid == 0)
                sh.csum[c2] = combine_slab_totals<NV>(s_sum, slab2);
        }
        __syncthreads();
    }
    /* where the draw falls: the same arithmetic in every workgroup of the row */
    if (tid < WAVE) {
        double    run, target;
        const int at = walk_locate_chunk(sh.csum, C, u_row, &run, &target);
        int       js = 0;
        if (at == chunk)
            js = walk_locate_slab<NV>(sh.slab, target, &run);
        if (tid == 0) {
            sh.walk.chunk    = at;
            sh.walk.slab     = js;
            sh.walk.before   = run;
            sh.walk.target   = target;
            sh.walk.pick     = 0x7fffffff;
            sh.walk.last_pos = -1;
        }
    }
    __syncthreads();
    if (sh.walk.chunk != chunk)
        return; /* another workgroup's */
    const double target = sh.walk.target;
    double       carry  = sh.walk.before;
    const int    js     = __builtin_amdgcn_readfirstlane(sh.walk.slab);
    int          end_w  = end;
    bool         found  = false;
    if (from_registers) {
        /* the located slab's weights, which the summation left in the registers: nothing is
         * computed again. Should rounding have left the target beyond the slab, the walk goes
         * on through the row from memory. */
        float4 vs = v[0];
#pragma unroll
        for (int j = 1; j < NV; ++j)
            if (j == js)
                vs = v[j];
        const int   sbase = base + js * 4 * TPB;
        const int   send  = sbase + 4 * TPB < end ? sbase + 4 * TPB : end;
        const int   e     = sbase + 4 * tid;
        const float w[4]  = {vs.x, vs.y, vs.z, vs.w};
        found = walk_slab_step<false>(w, e, send, target, carry, sh.walk);
        if (!found)
            walk_from<NV, PEN, false>(rv, row, n_rows, C, chunk, js + 1, carry, target, mx, inv_t,
                                      0.0, nullptr, false, -1, s_tab, s_cnt16, sh.walk, end_w);
    } else {
        walk_from<NV, PEN, false>(rv, row, n_rows, C, chunk, js, carry, target, mx, inv_t, 0.0,
                                  nullptr, false, -1, s_tab, s_cnt16, sh.walk, end_w);
    }
    __syncthreads();
    int tok = sh.walk.pick;
    if (tok == 0x7fffffff)
        tok = end_w - 1;
    if (tid == 0)
        out[row] = tok;
}

template <int NV, bool PEN>
__global__ __launch_bounds__(TPB) void k_temperature_draw(RowView rv, int n_rows, float inv_t,
                                                          const float *__restrict__ uniforms,
                                                          int32_t *__restrict__ out,
                                                          MeetSpace meet) {
    __shared__ __align__(16) uint32_t s_cnt16[PEN ? NV * TPB * 2 : 1];
    __shared__ double   s_sum[NWAVES * NV];
    __shared__ uint64_t s_tab[32];
    __shared__ uint64_t s_red[NWAVES], s_bb;
    __shared__ uint32_t s_arrive[2];
    __shared__ __align__(16) double s_tr_own[(NV == 8 && !PEN) ? NWAVES * 8 * WAVE : 1];
    __shared__ DrawShared s_draw;
    static_assert(!(NV == 8 && PEN) || sizeof(s_cnt16) >= NWAVES * 8 * WAVE * sizeof(double),
                  "the count table holds the transposed sums");
    double   *s_tr = PEN ? reinterpret_cast<double *>(s_cnt16) : s_tr_own;
    const int tid  = threadIdx.x;
    int       row, chunk;
    xcd_row_chunk(row, chunk);
    const uint64_t tabv = g_expf_tab[tid & 31];
    {
        const uint32_t wg = blockIdx.y * gridDim.x + blockIdx.x, n_wg = gridDim.x * gridDim.y;
        for (uint32_t i = wg * TPB + tid; i < meet.stale_count; i += n_wg * TPB)
            meet.stale[i] = 0;
    }
    if (row >= n_rows) /* the grid holds the rows in eights */
        return;
    int base, end;
    chunk_bounds<NV>(rv, chunk, base, end);
    FusedScan fs;
    fs.tmax       = nullptr;
    fs.chunk_best = nullptr;
    fs.slots      = meet.slots;
    fs.wait_limit = meet.wait_limit;
    fs.local      = meet.local;
    fs.s_red      = s_red;
    fs.s_bb       = &s_bb;
    fs.s_arrive   = s_arrive;
    uint64_t  *sum_slots = meet.slots + (long) n_rows * rv.n_chunks;
    const bool plain = rv.vec_ok && end - base == NV * TPB * 4 && !(rv.softcap > 0.0f) &&
                       rv.allowed == nullptr;
    if (plain)
        draw_chunk<NV, PEN, true>(rv, row, chunk, n_rows, base, end, inv_t, uniforms, out,
                                  sum_slots, s_cnt16, s_sum, s_tab, tabv, s_tr, s_draw, fs);
    else
        draw_chunk<NV, PEN, false>(rv, row, chunk, n_rows, base, end, inv_t, uniforms, out,
                                   sum_slots, s_cnt16, s_sum, s_tab, tabv, s_tr, s_draw, fs);
}

} // namespace gs
#endif
