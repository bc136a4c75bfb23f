// The per-wavefront ring of LDS slots that the matrix-core split-KV kernels (sdpa_decode_mfma.hip: f16 / bf16,
// sdpa_decode_f32.hip: f32) stream the key/value cache through: slot size, the non-temporal global -> LDS copy and
// the constant wait for the oldest copy in flight.
#pragma once
#include "sdpa_mfma_common.h"

namespace incin_rocm {

constexpr int DM_SLOT_BYTES = 8192;      // a block of K or of V: 16-bit storage 32 keys at D = 128, 64 at D = 64; f32 half as many
#ifndef DM_SHORT_KEYS
#define DM_SHORT_KEYS 2048      // (keys of 256 bytes: 16-bit storage at D = 128)
#endif
#ifndef DM_NSLOT
#define DM_NSLOT 5       // slots per wavefront: 4 wavefronts x 5 x 8 KiB = the 160 KiB of a compute unit
#endif

// One wavefront-wide global -> LDS copy of 64 x 16 bytes, as dma_copy16, marked non-temporal: every byte of the cache
// is read once per launch, and leaving it out of the caches' replacement order is worth 12 - 13 points of the memory
// bandwidth (measured on 32 x 32 heads x 8192 keys: 6.05 TB/s without the mark, 7.04 with it).
#ifndef DM_CACHE
#define DM_CACHE " nt"
#endif
__device__ __forceinline__ void dm_copy16(uint4v desc, unsigned lds_addr, int byte_offset)
{
    // (one wait state, as dma_copy16: the descriptors of these copies are put together right in front of them, and the build
    // checks the generated code)
    asm volatile(INCIN_DMA_WAIT "\n\tbuffer_load_dwordx4 %0, %1, 0 offen" DM_CACHE " lds" ::"v"(byte_offset), "s"(desc), "{m0}"(lds_addr) : "memory");
}

// All but the newest NSLOT - 1 copies of this wavefront (CPB instructions each: 8 for an 8 KiB slot) have landed.
template <int NSLOT, int CPB = 8> __device__ __forceinline__ void wait_oldest_copy()
{
    constexpr int N = (NSLOT - 1) * CPB;
    static_assert(N >= 1 && N <= 63, "s_waitcnt takes an immediate of 6 bits");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Which (batch entry, KV head, chunk of rows) a workgroup of the split-KV matrix-core kernels takes, from blockIdx.y and .z.
// With several chunks per KV head (prefill shapes through these kernels) the chunks of a head read the same keys and
// values: workgroups reach the 8 XCDs round-robin in dispatch order, so an unsplit launch hands each XCD a contiguous eighth
// of the list (a head's chunks then meet in one L2 instead of all eight), and the chunks of a head go last-first (under a
// causal mask the last rows see the most keys: longest first).
// longest_first (a causal launch of one query head per KV head, keys not split): the order is by length over the whole
// launch, not head by head - every (batch, head)'s last chunk, then every second-to-last, ... - because the workgroups that
// start last decide when the launch ends, and they should be the short ones; an XCD still keeps an eighth of the heads to itself.
// pairs: a compute unit holds two workgroups at a time, and the first two rounds of 32 per XCD all start at once - odd rounds
// go in reverse, so that a compute unit's pair is a long one and a short one.
__device__ __forceinline__ void decode_work_item(int nchunks, bool longest_first, bool pairs, int* b, int* hkv, int* chunk)
{
    int y = blockIdx.y;
    *b = blockIdx.z;
    if (nchunks > 1) {
        if (longest_first && gridDim.x == 1) {
            const int heads = (int)gridDim.y / nchunks, BH = (int)gridDim.z * heads;
            const int id = (int)blockIdx.z * (int)gridDim.y + y;      // dispatch order
            int bh, c;
            if ((BH & 7) == 0) {
                const int per = BH >> 3;
                int i = id >> 3;
                if (pairs && ((i >> 5) & 1)) {       // (the last round may be a partial one: reversed within what it has)
                    const int first = i & ~31, len = min(32, (BH * nchunks >> 3) - first);
                    i = first + (len - 1 - (i - first));
                }
                c = i / per;
                bh = (id & 7) * per + i % per;
            } else {
                c = id / BH;
                bh = id % BH;
            }
            *chunk = nchunks - 1 - c;
            *b = bh / heads;
            *hkv = bh % heads;
            return;
        }
        if (gridDim.x == 1 && (gridDim.y & 7) == 0) y = (y & 7) * (int)(gridDim.y >> 3) + (y >> 3);
        *hkv = y / nchunks;
        *chunk = nchunks - 1 - y % nchunks;
    } else {
        *hkv = y;
        *chunk = 0;
    }
}

}  // namespace incin_rocm
