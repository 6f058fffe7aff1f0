/* N-gram drafter for speculative decoding, one workgroup per sequence.
 *
 * The reference's propose_drafts_ngram (src/engine/session.c:437-513) looks for the longest
 * suffix of history + [seed], up to max_suffix tokens, that occurs earlier in the history; among
 * the occurrences of that length it prefers the one followed by the most tokens (counted up to
 * k_max - 1), the most recent one among equals, and proposes the tokens that followed it.
 *
 * Here every history position e < n - 1 is looked at once, as the place where the seed would
 * sit: m(e) = how many tokens ending at e agree with the suffix read backwards (seed,
 * h[n-1], h[n-2], ...), at most max_suffix and at most e + 1. The number of tokens that follow,
 * n - e - 1, does not depend on the suffix length, so the reference's nested search is one
 * maximum over a packed key: the match length first; then whether k_max - 1 tokens follow
 * (e <= n - k_max), and among those the largest e; otherwise the smallest e (the most that
 * follow). A position with m(e) >= L is a candidate of every shorter length too, but the
 * reference stops at the first length that has any, which is max m. */
#pragma once
#include "sampler_device.h"
#include "sampler_kernels.h"

namespace gs {

__global__ __launch_bounds__(TPB) void k_ngram_draft(const int32_t *__restrict__ history,
                                                     long history_ld,
                                                     const int32_t *__restrict__ history_len,
                                                     const int32_t *__restrict__ seeds, int k_max,
                                                     int max_suffix, int32_t *__restrict__ out,
                                                     long out_ld, int32_t *__restrict__ out_count,
                                                     int32_t *__restrict__ out_match) {
    __shared__ uint64_t s_red[NWAVES];
    const int           seq = blockIdx.x, tid = threadIdx.x;
    const int32_t      *h   = history + (long) seq * history_ld;
    const int           n   = history_len[seq] > 0 ? history_len[seq] : 0;
    const int32_t       sd  = seeds[seq];
    int32_t            *o   = out + (long) seq * out_ld;
    const int           cap = max_suffix > NGRAM_SUFFIX_MAX ? NGRAM_SUFFIX_MAX : max_suffix;
    /* the suffix read backwards; entries that would lie before the history are never compared,
     * because m(e) <= e + 1 <= n - 1 */
    int32_t suffix[NGRAM_SUFFIX_MAX];
    suffix[0] = sd;
#pragma unroll
    for (int j = 1; j < NGRAM_SUFFIX_MAX; ++j)
        suffix[j] = n - j >= 0 ? h[n - j] : -1;
    uint64_t best = 0;
    if (k_max > 1 && cap >= 1) {
        for (int e = tid; e < n - 1; e += TPB) {
            if (h[e] != sd)
                continue;
            int m = 1;
#pragma unroll
            for (int j = 1; j < NGRAM_SUFFIX_MAX; ++j) {
                if (m != j || j >= cap || e - j < 0 || h[e - j] != suffix[j])
                    continue;
                m = j + 1;
            }
            const bool     full = e <= n - k_max;
            const uint64_t key  = ((uint64_t) m << 40) |
                                 (full ? (1ull << 39) | (uint64_t) e : (uint64_t) (0x7fffffff - e));
            best = key > best ? key : best;
        }
    }
    best = block_max_u64(best, s_red);
    int count = 1, match = 0;
    if (best) {
        match            = (int) (best >> 40);
        const bool full  = (best >> 39) & 1;
        const int  low   = (int) (best & 0x7fffffffu);
        const int  e     = full ? low : 0x7fffffff - low;
        const int  avail = n - e - 1;
        const int  take  = avail < k_max - 1 ? avail : k_max - 1;
        if (tid < take)
            o[1 + tid] = h[e + 1 + tid];
        count = 1 + take;
    }
    if (tid == 0) {
        o[0]           = sd;
        out_count[seq] = count;
        out_match[seq] = match;
    }
}

} // namespace gs
