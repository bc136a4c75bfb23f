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
    asm volatile("s_nop 0\n\tbuffer_load_dwordx4 %0, %1, 0 offen" DM_CACHE " lds" ::"v"(byte_offset), "s"(desc), "{m0}"(lds_addr) : "memory");
}

// All but the newest NSLOT - 1 copies of this wavefront (CPB instructions each: 8 for an 8 KiB slot) have landed.
template <int NSLOT, int CPB = 8> __device__ __forceinline__ void wait_oldest_copy()
{
    constexpr int N = (NSLOT - 1) * CPB;
    static_assert(N == 8 || N == 16 || N == 24 || N == 32, "s_waitcnt takes an immediate");
    if (N == 32) asm volatile("s_waitcnt vmcnt(32)" ::: "memory");
    else if (N == 24) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
    else if (N == 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
}

// Which (KV head, chunk of rows) a workgroup of the split-KV matrix-core kernels takes, from blockIdx.y.  With several
// chunks per KV head (prefill shapes through these kernels) the chunks of a head read the same keys and values: workgroups
// reach the 8 XCDs round-robin in dispatch order, so an unsplit launch hands each XCD a contiguous eighth of the list
// (a head's chunks then meet in one L2 instead of all eight), and the chunks of a head go last-first (under a causal
// mask the last rows see the most keys: longest first).
__device__ __forceinline__ void decode_work_item(int nchunks, int* hkv, int* chunk)
{
    int y = blockIdx.y;
    if (nchunks > 1) {
        if (gridDim.x == 1 && (gridDim.y & 7) == 0) y = (y & 7) * (int)(gridDim.y >> 3) + (y >> 3);
        *hkv = y / nchunks;
        *chunk = nchunks - 1 - y % nchunks;
    } else {
        *hkv = y;
        *chunk = 0;
    }
}

}  // namespace incin_rocm
