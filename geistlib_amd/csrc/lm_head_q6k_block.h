/* A Q6_K super-block as it lies in a GGUF file (src/quant/quant_blocks.h:67-73: ql[128], qh[64],
 * sixteen int8 scales, one binary16 d; 210 bytes, 2-byte aligned), read by one lane. Shared by the
 * kernels that read the table without a packed copy. */
#ifndef GEIST_LM_HEAD_Q6K_BLOCK_H
#define GEIST_LM_HEAD_Q6K_BLOCK_H

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gs {

typedef uint32_t q6k_u32x4 __attribute__((ext_vector_type(4), aligned(4)));

/* The 53 dwords of the block at `bp` (2-byte aligned), shifted into place: d[0..31] ql,
 * d[32..47] qh, d[48..51] the scales, the low half of d[52] the binary16 d. The aligned dwords
 * that hold the block are read whole; what they hold beyond the block lies in the same aligned
 * dword as a byte of the block, so no load leaves the table's pages. */
__device__ __forceinline__ void q6k_load_block(const uint8_t *bp, uint32_t (&d)[53]) {
    const uintptr_t a     = reinterpret_cast<uintptr_t>(bp);
    const uint32_t  shift = (uint32_t) (a & 2) * 8; /* 0 or 16 */
    const uint32_t *p     = reinterpret_cast<const uint32_t *>(a & ~(uintptr_t) 3);
    uint32_t        raw[54];
#pragma unroll
    for (int i = 0; i < 52; i += 4) {
        const q6k_u32x4 q = *reinterpret_cast<const q6k_u32x4 *>(p + i);
        raw[i] = q.x, raw[i + 1] = q.y, raw[i + 2] = q.z, raw[i + 3] = q.w;
    }
    raw[52] = p[52];
    raw[53] = 0u; /* (only the low half of d[52] is used, and raw[52] holds it either way) */
#pragma unroll
    for (int i = 0; i < 53; ++i)
        d[i] = __builtin_amdgcn_alignbit(raw[i + 1], raw[i], shift);
}

} // namespace gs
#endif
