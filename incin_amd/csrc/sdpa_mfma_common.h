// Shared pieces of the MFMA attention kernels: operand types, the matrix
// instruction wrappers, the LDS tile layout (chunk-slot swizzle) and the
// lane <-> lane^32 exchanges.
#pragma once
#include <atomic>

#include "sdpa_params.h"

namespace incin_rocm {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));
typedef bf16_t bf16x8 __attribute__((ext_vector_type(8)));
typedef f16_t f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));

template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
    typedef bf16x8 vec8;
    typedef bf16_t vec2 __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ floatx16 run(vec8 a, vec8 b, floatx16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    // acc + x[0] + x[1] (f32 accumulate of the two storage-precision values)
    static __device__ __forceinline__ float add2(vec2 x, float acc)
    {
        const vec2 ones = {(bf16_t)1.0f, (bf16_t)1.0f};
        return __builtin_amdgcn_fdot2_f32_bf16(x, ones, acc, false);
    }
};
template <> struct Mma<f16_t> {
    typedef f16x8 vec8;
    typedef f16_t vec2 __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ floatx16 run(vec8 a, vec8 b, floatx16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float add2(vec2 x, float acc)
    {
        const vec2 ones = {(f16_t)1.0f, (f16_t)1.0f};
        return __builtin_amdgcn_fdot2(x, ones, acc, false);
    }
};

constexpr int PF_BM = 128;     // query rows per workgroup
constexpr int PF_BN = 64;      // keys per tile
constexpr float PF_RESCALE_THRESHOLD = 8.0f;   // log2 units

template <int D> struct PfLayout {
    static constexpr int ROWB = D * 2;                 // bytes per K/V row in LDS (unpadded)
    static constexpr int CPR = D / 8;                  // 16-byte chunks per row
    static constexpr int TILE_BYTES = PF_BN * ROWB;    // one K or V tile
    static constexpr int STAGE_BYTES = 2 * TILE_BYTES; // K then V
    static constexpr int LOADS_PER_WAVE = TILE_BYTES / 1024 / 4;   // wavefront-wide 1 KiB loads per tensor per tile
    // Chunk-slot swizzles (functions of the low 4 bits of the row).
    // K tile: read by 16 lanes x 16 bytes down 16 consecutive rows at one logical chunk, so fk must
    // take 16 distinct values over 16 consecutive rows (D = 64: 8 distinct over rows of one parity,
    // because two 128-byte rows already split the banks).
    static __device__ __forceinline__ int fk(int r)
    {
        if (D >= 128) return ((r & 3) << 2) | ((r >> 2) & 3);
        return (((r >> 1) & 1) << 2) | ((r >> 2) & 3);
    }
    // V tile: the transposing read takes 4 consecutive rows x 64 bytes per half-wavefront, so fv only
    // has to move those 4 rows to 4 different 64-byte column groups; keeping it a function of row
    // bits 0-1 (D = 64: bit 1) makes the read address base ^ (d_block << 6) + immediate.
    static __device__ __forceinline__ int fv(int r)
    {
        if (D >= 128) return (r & 3) << 2;
        return ((r >> 1) & 1) << 2;
    }
};

// The same for rows of f32 (the IEEE-f32 kernels: sdpa_prefill_f32.hip, sdpa_decode_f32.hip).
template <int D> struct F32Layout {
    static constexpr int ROWB = D * 4;                       // bytes per K/V row in LDS (unpadded)
    static constexpr int CPR = D / 4;                        // 16-byte chunks per row
    static constexpr int TILE_BYTES = 16384;
    static constexpr int KT = TILE_BYTES / ROWB;             // keys per tile: 64 (D = 64), 32 (D = 128)
    static constexpr int NB = KT / 32;                       // 32-key blocks per tile
    static constexpr int LOADS_PER_WAVE = TILE_BYTES / 1024 / 4;
    // Chunk c of row r sits at chunk c ^ f(r).  K reads go down 16 consecutive rows at one logical chunk: f takes 16
    // values there.  V reads take rows r and r + 4 (r % 8 < 4) in the two halves of a wavefront, eight consecutive
    // chunks each: f(r) and f(r + 4) differ in bit 3, which sends the halves to different halves of the banks.
    static __device__ __forceinline__ int f(int r) { return (r & 3) | ((r & 4) << 1) | ((r & 8) >> 1); }
};

// One wavefront-wide global -> LDS copy (64 lanes x 16 bytes land at lds_addr .. lds_addr + 1023 in lane order; lanes
// whose offset is outside the descriptor's range deliver zeros).  Issued through inline assembly on purpose: the
// compiler makes every LDS access it cannot prove disjoint from a copy it knows of wait until that copy has landed -
// for the transposing reads that is a full memory latency in the middle of every tile - whereas the kernels here
// order copies and reads themselves (s_waitcnt vmcnt + barrier before a buffer is read, a barrier after its last read
// before it is refilled).  Counting the copy in vmcnt stays correct for the compiler's own loads: memory operations
// complete in order, so its waits only become stricter.
__device__ __forceinline__ uint4v dma_descriptor(const void* base, int bytes)
{
    const unsigned long long a = (unsigned long long)base;
    const uint4v d = {(unsigned)a, (unsigned)(a >> 32) & 0xffffu, (unsigned)bytes, 0x00020000u};
    return d;
}
__device__ __forceinline__ unsigned lds_address(const void* p)
{
    return (unsigned)(unsigned long long)(const __attribute__((address_space(3))) char*)p;
}
// Wait states in front of a copy.  One is what a write of m0 needs before the copy that reads it.  Five is what a vector
// instruction that wrote one of the copy's scalar operands needs: the compiler brings spilled scalar registers back with
// v_readlane_b32, may do so right in front of the statement, does not see the memory instruction inside it and so adds no
// wait states itself - and a copy that read a stale descriptor has fetched from wherever that pointed (wrong values, or a
// memory fault).  The copies of the K / V / Q / dO tiles, whose descriptors are put together by scalar instructions right
// in front of them, keep one wait state (five cost the prefill kernel 0.5 - 1 %), and the build checks the code the compiler
// wrote for every such copy (incin_amd/hazards.py: it fails if a vector write of an operand is nearer than five wait states);
// the others (descriptors that live across a kernel and may come back from a spill) take five.
#ifndef INCIN_DMA_WAIT
#define INCIN_DMA_WAIT "s_nop 0"
#endif
__device__ __forceinline__ void dma_copy16(uint4v desc, unsigned lds_addr, int byte_offset)
{
    asm volatile(INCIN_DMA_WAIT "\n\tbuffer_load_dwordx4 %0, %1, 0 offen lds" ::"v"(byte_offset), "s"(desc), "{m0}"(lds_addr) : "memory");
}
// The same with a wavefront-uniform byte offset added to every lane's (the instruction's scalar offset operand): copies that
// differ only by such an offset share one register of lane offsets.
__device__ __forceinline__ void dma_copy16_at(uint4v desc, unsigned lds_addr, int byte_offset, int uniform_offset)
{
    asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds" ::"v"(byte_offset), "s"(desc), "s"(uniform_offset), "{m0}"(lds_addr) : "memory");
}
// Offset for the lane of such a copy that fetches 16-byte chunk `chunk` of row `row` (rows `row_bytes` apart in memory,
// `data_bytes` of data each): a chunk at or beyond the row's data gets an offset that no descriptor covers, so that lane
// delivers zeros.  This is how a head dimension below the one a kernel instance is built for is padded: with zeros, on
// the way into LDS, without touching the operands in memory.
__device__ __forceinline__ int dma_chunk_offset(int row, int row_bytes, int chunk, int data_bytes)
{
    return chunk * 16 < data_bytes ? row * row_bytes + chunk * 16 : 0x7fffffff;
}
// The same for 64 lanes x 4 bytes (256 bytes of LDS).
__device__ __forceinline__ void dma_copy4(uint4v desc, unsigned lds_addr, int byte_offset)
{
    asm volatile("s_nop 4\n\tbuffer_load_dword %0, %1, 0 offen lds" ::"v"(byte_offset), "s"(desc), "{m0}"(lds_addr) : "memory");
}

// CU count of the current device (256 if the query fails: only launch geometry depends on it).
inline int device_cus()
{
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

// ---- order of the work list ------------------------------------------------------------------------------------
// A work item is (batch, KV head, query head of its group, block of query rows).  The list runs over groups of F
// (batch, KV head) pairs; inside a group the query blocks go longest-first (under a causal mask the last block sees
// the most keys), and for each block all F * G heads of the group follow one another.  With F * G * (blocks per head)
// a multiple (twice, measured best) of the workgroups an XCD runs at a time, every round of workgroups gets items of
// nearly equal length, which
// list scheduling in plain head order does not give (it ends each head on its shortest blocks while the next head's
// longest start, and the last round is left ragged: about 9 % at 4096 x 4096 causal).  F is kept small: F KV heads
// are in an XCD's L2 at a time.
struct WorkItem { int bhkv, gq, qblk; };
__device__ __forceinline__ WorkItem work_item(int vid, int F, int G, int nqb)
{
    const int per_group = F * G * nqb;
    const int grp = vid / per_group, r = vid - grp * per_group;
    const int rank = r / (F * G), m = r - rank * (F * G);
    WorkItem w;
    w.bhkv = grp * F + m / G;
    w.gq = m % G;
    w.qblk = nqb - 1 - rank;
    return w;
}
// Item `item` of XCD `xcd`'s share of the work list (a share holds share_len items).  When a share holds whole
// groups, (batch, KV head) pairs are dealt to the XCDs in turn - pair h goes to XCD h % 8, and an XCD groups the
// pairs it holds F at a time - so the sequences of a ragged batch spread over all XCDs instead of one long sequence
// filling the shares of two of them.  Otherwise a share is a contiguous eighth of the list - unless (deal = 2) a share is
// less than one group and the group's blocks differ in length (a causal mask): a contiguous piece of a list that runs
// longest-first would give one XCD the long blocks of every head and another the short ones (8 query heads on one KV head,
// 64 blocks each: the first XCD would get 1.9 times the average), so the list is dealt item by item - item i of the list to
// XCD i % 8, which is the order workgroups reach the XCDs in anyway.
__device__ __forceinline__ WorkItem work_item_of_share(int xcd, int item, int share_len, int F, int G, int nqb, int deal)
{
    if (deal == 2) return work_item(item * 8 + xcd, F, G, nqb);
    if (!deal) return work_item(xcd * share_len + item, F, G, nqb);
    const int per_group = F * G * nqb;
    const int g_local = item / per_group, r = item - g_local * per_group;
    const int rank = r / (F * G), m = r - rank * (F * G);
    WorkItem w;
    w.bhkv = (g_local * F + m / G) * 8 + xcd;
    w.gq = m % G;
    w.qblk = nqb - 1 - rank;
    return w;
}
inline int work_deal(int F, int G, int nqb, long long share_items, bool uneven)
{
    const long long group = (long long)F * G * nqb;
    // (item by item only where a share is less than a group - the few heads of such a launch fit the last-level cache whichever
    //  XCD reads them.  With more heads than XCDs the contiguous shares keep a head's K and V in one L2, and dealing such lists
    //  item by item loses more than the ragged shares cost: 12 heads x 8192 keys 932 -> 772 TFLOP/s, 5 x 12 heads x 4096 929 -> 734.)
    return share_items % group == 0 ? 1 : (uneven && share_items < group ? 2 : 0);
}

// F for a launch: `slots` workgroups run on an XCD at a time, a range of the list (the whole list, or an eighth of it
// when it divides by 8 and each XCD takes one) holds `range_items` items.
// (`causal`: the blocks of a head differ in length - a causal flag, or a mask tensor, which more often than not is a causal
// mask; with blocks of equal length the interleaved order costs nothing)
inline int work_interleave(bool causal, int slots, int G, int nqb, long long range_items)
{
    if (!causal || slots <= 0) return 1;
    int a = slots, b = (G * nqb) % slots;
    while (b) { const int t = a % b; a = b; b = t; }          // a = gcd(slots, G * nqb)
    int f = 2 * (slots / a);          // two rounds per group: a slot that drew a long block first draws a short one next
    if (f > 8) f = 8;
    while (f > 1 && range_items % ((long long)f * G * nqb)) --f;
    return f;
}

// ---- Q rows in, O rows out: 16 bytes per lane, eight lanes to a 128-byte run of a row -------------------------------
// The prefill kernels keep a query per lane: lane (ql, g) of a wavefront holds, of row ql, the 16-byte chunks
// 2 s + g of Q (one per k-step s; f32: per group of four k-steps) and of O the four columns db * 32 + r4 * 8 + g * 4 ..
// per (db, r4).  Read and written
// that way, every memory instruction touches 32 rows with 16 or 32 bytes each, and the compute unit's path to memory takes
// such partial cache lines one at a time (512 of them per wavefront for 64 lines of data).  So both go through a
// wavefront-private 4 KiB of LDS, 128 bytes per row (64 columns, 32 in f32) per pass: chunk c of row r at chunk c ^ (r % 8).  Both are
// non-temporal: rows that are used once must not push the K / V tiles, which every workgroup of a head reads, out of L2.
// No barrier is involved: the area belongs to one wavefront; the caller says which LDS nobody else touches meanwhile.
template <typename T, int NQH>
__device__ __forceinline__ void fetch_q_rows(uint4v (&qraw)[NQH][4], const T* qhead, int row0, int Sq, int64_t q_ss, int Dq, int lane)
{
#pragma unroll
    for (int h = 0; h < NQH; ++h)
#pragma unroll
        for (int ps = 0; ps < 4; ++ps) {
            const int rr = ps * 8 + (lane >> 3), col = h * (int)(128 / sizeof(T)) + (lane & 7) * (int)(16 / sizeof(T));
            const uint4v zero = {0u, 0u, 0u, 0u};
            // (rows past the last one repeat it: their results are never stored; beyond the head dimension: zeros, like K's)
            qraw[h][ps] = col < Dq ? __builtin_nontemporal_load((const uint4v*)(qhead + (int64_t)min(row0 + rr, Sq - 1) * q_ss + col)) : zero;
        }
}
// (NS k-steps' worth of operands are taken out: 4 * NQH, or fewer when the last columns of the last pass are padding)
template <typename V8, int NS, int NQH>
__device__ __forceinline__ void stage_q_rows(V8 (&qreg)[NS], const uint4v (&qraw)[NQH][4], char* stage, int lane)
{
    const int ql = lane & 31, g = lane >> 5;
#pragma unroll
    for (int h = 0; h < NQH; ++h) {
#pragma unroll
        for (int ps = 0; ps < 4; ++ps) {
            const int rr = ps * 8 + (lane >> 3), c = lane & 7;
            *(uint4v*)(stage + rr * 128 + ((c ^ (rr & 7)) << 4)) = qraw[h][ps];
        }
#pragma unroll
        for (int sl = 0; sl < 4; ++sl)
            if (h * 4 + sl < NS) qreg[h * 4 + sl] = *(const V8*)(stage + ql * 128 + (((2 * sl + g) ^ (ql & 7)) << 4));
    }
}
template <typename T, int NDB>
__device__ __forceinline__ void store_o_rows(const floatx16 (&o_acc)[NDB], float inv, char* stage, T* ohead, int row0, int rows_b, int64_t o_ss, int Dv, int lane)
{
    typedef T vec4 __attribute__((ext_vector_type(4)));
    const int ql = lane & 31, g = lane >> 5;
#pragma unroll
    for (int h = 0; h < (NDB + 1) / 2; ++h) {      // (an odd NDB: the last pass is half full, and Dv cuts its stores)
#pragma unroll
        for (int dbl = 0; dbl < 2 && 2 * h + dbl < NDB; ++dbl)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                vec4 w;
#pragma unroll
                for (int e = 0; e < 4; ++e) w[e] = (T)(o_acc[2 * h + dbl][r4 * 4 + e] * inv);
                *(vec4*)(stage + ql * 128 + (((dbl * 4 + r4) ^ (ql & 7)) << 4) + g * 8) = w;
            }
#pragma unroll
        for (int ps = 0; ps < 4; ++ps) {
            const int rr = ps * 8 + (lane >> 3), c = lane & 7;
            const uint4v val = *(const uint4v*)(stage + rr * 128 + ((c ^ (rr & 7)) << 4));
            const int col = h * 64 + c * 8;
            if (row0 + rr < rows_b && col < Dv) __builtin_nontemporal_store(val, (uint4v*)(ohead + (int64_t)(row0 + rr) * o_ss + col));
        }
    }
}

// (f32: a pass is one 32-column block; the lane's four floats of (db, r4) are chunk 2 r4 + g of it)
template <int NDB>
__device__ __forceinline__ void store_o_rows_f32(const floatx16 (&o_acc)[NDB], float inv, char* stage, float* ohead, int row0, int rows_b, int64_t o_ss, int Dv, int lane)
{
    typedef float f4 __attribute__((ext_vector_type(4)));
    const int ql = lane & 31, g = lane >> 5;
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            f4 w;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = o_acc[db][r4 * 4 + e] * inv;
            *(f4*)(stage + ql * 128 + (((2 * r4 + g) ^ (ql & 7)) << 4)) = w;
        }
#pragma unroll
        for (int ps = 0; ps < 4; ++ps) {
            const int rr = ps * 8 + (lane >> 3), c = lane & 7;
            const uint4v val = *(const uint4v*)(stage + rr * 128 + ((c ^ (rr & 7)) << 4));
            const int col = db * 32 + c * 4;
            if (row0 + rr < rows_b && col < Dv) __builtin_nontemporal_store(val, (uint4v*)(ohead + (int64_t)(row0 + rr) * o_ss + col));
        }
    }
}

__device__ __forceinline__ float xor32_max(float x)
{
    // lanes l and l^32 exchange; both end with the maximum
    auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
}

__device__ __forceinline__ float xor32_sum(float x)
{
    auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
}

}  // namespace incin_rocm
