// bf16 / f16 attention forward on the gfx950 matrix cores (prefill shapes).
//
// Computes the function of the reference CPU composition
// (crates/incin-backends/src/cpu/ops/shape_ops.rs:1245-1269) for head dimensions up to 128 (instances for 64 and
// 128; a smaller D or Dv, in whole 16-byte vectors, is zero-padded on the way into LDS and the stores are cut at Dv),
// optional causal mask and per-batch key lengths, MHA and GQA, with
// f32 accumulation and an online softmax: no score tensor is ever materialised.
//
// Shape of the computation (one workgroup = 4 wavefronts = 128 query rows, one
// wavefront = 32 query rows, key tile = 64 keys):
//
//   S^T = K_tile Q'^T    v_mfma_f32_32x32x16: A = K rows from LDS (16-byte reads),
//                        B = Q^T held in registers for the whole kernel, already
//                        multiplied by scale*log2(e).  In the 32x32 result a lane
//                        owns ONE query (column lane%32) and 16 keys per 32-key
//                        block, so the row max and row sum of the softmax are
//                        in-lane reductions plus one exchange with lane^32.  The
//                        accumulator starts from -m_ref (the lane's reference
//                        maximum) instead of 0, so the product already is s - m.
//   P^T                  a bare exp2 of that, rounded to the storage type in
//                        registers; the accumulator layout of S^T is already the
//                        B-operand layout of the next product (the key order inside
//                        a k-step is a fixed permutation, which the V reads follow).
//   O^T += V^T P^T       A = V^T read from the row-major V tile in LDS with the
//                        transposing LDS read (ds_read_b64_tr_b16).
//
// Data movement: K and V tiles go from global memory straight into LDS
// (buffer_load ... lds, 16 bytes per lane, no register staging) into two
// alternating buffers each; out-of-range rows are zero-filled by the buffer
// descriptor's bounds check.  LDS rows are unpadded; the 16-byte chunk c of row r
// is stored at chunk slot c ^ f(r), with f chosen per tile kind so that both read
// patterns (16 lanes x 16 bytes down a column of rows for K; 4 rows x 64 bytes
// for the transposing V read) touch every bank once.
//
// Overlap: the vector ALU work of the softmax and the matrix instructions of a wavefront only run
// side by side when they are interleaved in that wavefront's own instruction stream (instructions of
// the two wavefronts that share a SIMD take turns instead).  So the kernel is software-pipelined over
// key tiles: while the matrix pipe computes S^T(t+1), the vector ALU turns S^T(t) into P^T(t) (two
// exponentials, one pack per MFMA; the order is pinned with scheduling group barriers), and while the
// matrix pipe computes O^T += V(t)^T P(t)^T the vector ALU takes the maxima of S^T(t+1).  Two score
// tiles are alive at a time.  This loop runs over the tiles that need no mask; a wavefront's last
// tiles (the diagonal ones of a causal mask, the ragged end of a key length) go through a plain
// one-tile-at-a-time loop with masking.
//
// One barrier per tile, at the top of the iteration: it publishes K(t+1) and V(t), whose global loads
// were started one iteration earlier, and frees the buffers of K(t) and V(t-1), into which the loads
// of K(t+2) and V(t+1) start right away.  Matrix operands are read from LDS a few MFMAs ahead of use.
//
// The reference maximum is set from the first tile that holds a visible key and
// afterwards only raised when a tile's maximum exceeds it by more than 2^8 (the
// accumulator and the running sum are rescaled then); otherwise probabilities
// are taken against the stale maximum, which is exact in exact arithmetic and
// keeps every intermediate within f32 / storage range.
//
// bf16 without a dense mask goes one step further in the pipelined loop and takes no maxima there at
// all.  bf16 has the exponent range of f32, so the probabilities are carried 2^-64 times smaller
// (the reference is kept 64 above the maximum it was taken from) and the only thing to know about a
// tile is whether some probability reached 2.0 - bit 14 of a bf16 - i.e. whether a score passed the
// stale maximum by more than 2^64: the packed probabilities are OR-ed together as they are made
// (8 instructions per tile instead of 21 for the maxima) and one test of the result decides.  If the
// bit is set, the exact path runs before anything of that tile is accumulated: maximum of the tile,
// reference raised, O^T and the row sum rescaled, the probabilities taken again.  Scores more than
// 2^62 below the reference flush to zero, which is far below what bf16 resolves.  The vector ALU
// instructions saved are the point: on N(0,1) inputs this kernel is limited by power (the same
// launch on zero inputs runs 1.4 times faster), and every instruction not issued is clock gained.
#include <cstdlib>
#include <type_traits>

#include "sdpa_mfma_common.h"

namespace incin_rocm {

#ifndef PF_KD
#define PF_KD 2     // K operand reads run this many k-steps ahead of their MFMAs
#endif
#ifndef PF_VD
#define PF_VD 4     // V operand reads run this many MFMAs ahead
#endif

// NW wavefronts = 32 * NW query rows per workgroup: 4 (two workgroups per compute unit) or 8 (one, whose K / V tiles then
// serve 256 rows: half the global -> LDS copies per matrix instruction).
//
// SPLIT: the launch is a grid of (work items) x (splits of the key axis); a workgroup handles the keys of its split only and
// writes, per row, the unnormalised O, the reference and the sum - the partial-result format of the split-KV kernels, whose
// combine kernel finishes the job.  For launches with too few (batch, head, row block) items to fill the device over a long
// key axis (a chunk of a long prompt, a single sequence): the key axis supplies the parallelism the rows lack.
//
// KS, NB: the k-steps of 16 head-dimension columns the score product runs over, and the 32-column blocks of the output it
// keeps.  D fixes the layout of a tile in LDS (rows of D columns, zero beyond the tensors' own); head dimensions that fill only
// part of it leave the rest out of the arithmetic as well: 6 k-steps and 3 blocks for head dimensions up to 96 in the 128 layout.
//
// MASK: 0 no mask tensor; 1 (DENSE) a dense additive mask, by block flags and values; 2 (LIMS) a launch with a dense mask for
// the workgroups all of whose rows the mask gives n zeros and then -inf (mask_row_limits_kernel wrote n per row: a causal mask,
// key padding, both): to them the tensor says nothing their limits do not, and they run exactly as without one.  A masked
// request is two launches, LIMS then DENSE, and every block of p.lims_rows rows is computed by one of them: by LIMS if all
// its rows have a limit, else by DENSE (whose workgroups look at the limits of the LIMS block, or blocks, that hold their rows).
// 3 (STAGED) is DENSE with the mask's values brought into LDS: every wavefront copies the 32 rows x 64 keys of its own rows a
// tile ahead, with the K and V copies of that tile, into one of two 4 KiB buffers of its own (16-byte chunks XOR-swizzled by
// row so that the 8-byte reads of a wavefront meet no bank conflict), and takes them from there.  A value loaded from memory
// inside a tile would make the compiler wait for everything in flight - the next tiles' copies, which it does not know of,
// included - a memory latency in every tile; and there are no registers to hold a tile's values a tile ahead.
template <typename T, int D, int MASK, int NW, bool SPLIT = false, int KS = D / 16, int NB = D / 32>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(2, 2)))
void sdpa_prefill_mfma_kernel(SdpaParams p)
{
    constexpr bool STAGED = MASK == 3, DENSE = MASK == 1 || STAGED, LIMS = MASK == 2;
#if defined(__HIP_DEVICE_COMPILE__)   // the body uses device-only types (buffer descriptors); the host pass needs only the stub
    typedef typename Mma<T>::vec8 vec8;
    typedef PfLayout<D> L;
    constexpr int NSTEP = KS;              // k-steps of the S^T product
    constexpr int NDB = NB;                // 32-wide blocks of the head dimension
    static_assert(KS <= D / 16 && NB <= D / 32 && KS >= 4 && NB >= 1, "");
    // the 8 slices of 4 scores a tile's probabilities are taken in, dealt over the k-steps of the next tile's score product
    // (slices slice_lo(s) .. slice_lo(s + 1) - 1 under k-step s), and the 16 pairs of the row sum (or the 16 registers of
    // the maximum) over the MFMAs of the O^T update
    auto slice_lo = [](int s) constexpr { return s * 8 / KS; };
    auto pair_lo = [](int i) constexpr { return i * 16 / (4 * NB); };
    constexpr int LPW = L::TILE_BYTES / 1024 / NW;     // wavefront-wide 1 KiB copies per tensor per tile
    constexpr int BM = 32 * NW;                        // query rows per workgroup
    // bf16 without a dense mask: probabilities are taken 2^-SHIFT times smaller, so that "some probability reached 2"
    // - one bit of the packed values - says that a score passed the reference by more than 2^SHIFT
    constexpr bool BF16 = std::is_same<T, bf16_t>::value;
    constexpr bool ORCHK = BF16 && !DENSE;
    constexpr float SHIFT = BF16 ? 64.0f : 0.0f;

    __shared__ __attribute__((aligned(1024))) char smem[4 * L::TILE_BYTES];   // K buffers 0, 1, V buffers 0, 1

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);     // wavefront-uniform by construction: keep it scalar
    const int ql = lane & 31, g = lane >> 5;
    const int Sq = p.Sq, Skv = p.Skv;

    // ---- which (batch, head, query block) -----------------------------------
    // Workgroups reach the 8 XCDs round-robin by id; hand each XCD a contiguous
    // range of the work list so heads that share K/V stay in one L2.
    const int nqb = (Sq + BM - 1) / BM;
    const int total = gridDim.x;
    const WorkItem wi = (total & 7) == 0 ? work_item_of_share(blockIdx.x & 7, blockIdx.x >> 3, total >> 3, p.interleave, p.G, nqb, p.deal_groups)
                                         : work_item(blockIdx.x, p.interleave, p.G, nqb);
    const int gq = wi.gq, qb = wi.qblk, bhkv = wi.bhkv;
    const int hkv = bhkv % p.Hkv, b = bhkv / p.Hkv;
    const int hq = hkv * p.G + gq;
    const int q0 = qb * BM;

    const T* qp = (const T*)p.q + (int64_t)b * p.q_sb + (int64_t)hq * p.q_sh;
    const T* kp = (const T*)p.k + (int64_t)b * p.k_sb + (int64_t)hkv * p.k_sh;
    const T* vp = (const T*)p.v + (int64_t)b * p.v_sb + (int64_t)hkv * p.v_sh;
    T* op = (T*)p.o + (int64_t)b * p.o_sb + (int64_t)hq * p.o_sh;

    int kv_len = Skv;
    if (p.kv_lens) kv_len = clampi(p.kv_lens[b], 0, Skv);
    // a split ends where the next begins: to this workgroup the keys beyond do not exist (split_len is a multiple of two tiles)
    const int split = SPLIT ? (int)blockIdx.y : 0;
    if (SPLIT) kv_len = min(kv_len, (split + 1) * p.split_len);
    // query rows at and beyond rows_b are padding: nothing is computed or stored for them
    const int rows_b = p.q_lens ? clampi(p.q_lens[b], 0, Sq) : Sq;
    if (q0 >= rows_b) return;                          // the whole block is padding (uniform: before any barrier)
    const int coff = Skv - Sq;
    // keys visible to this workgroup / this wavefront / this lane's query
    int j_end = kv_len;
    const int my_i = q0 + wave * 32 + ql;
    int lim_lane = kv_len, lim_wave_min = kv_len, lim_wave_max = kv_len;
    if (p.causal) {
        const int last_row = min(q0 + BM - 1, rows_b - 1);
        j_end = clampi(last_row + coff + 1, 0, kv_len);
        lim_lane = clampi(my_i + coff + 1, 0, kv_len);
        lim_wave_min = clampi(q0 + wave * 32 + coff + 1, 0, kv_len);
        lim_wave_max = clampi(min(q0 + wave * 32 + 31, rows_b - 1) + coff + 1, 0, kv_len);
    }
    if (q0 + wave * 32 >= rows_b) lim_wave_min = lim_wave_max = 0;      // a wavefront of padding rows only keeps the barriers company
    int n_tiles = (j_end + PF_BN - 1) / PF_BN;
    // ---- dense additive mask: what its block flags say about this workgroup's rows ---------------------------------
    // mflags: one byte per 32-key block for this wavefront's 32 rows (0 mixed, 1 all zero, 2 all -inf).  Tiles before
    // the first and after the last one in which some wavefront has a visible block are never copied; in between, a
    // wavefront skips the tiles hidden from its own rows.
    const uint8_t* mflags = nullptr;
    const T* mrow = nullptr;
    const int nkb32 = (Skv + 31) >> 5;
    int t_first = SPLIT ? min(split * (p.split_len / PF_BN), n_tiles) : 0;
    [[maybe_unused]] int w_first = 0, w_last = 0x7fffffff;      // this wavefront's first and last tile with a visible block
    [[maybe_unused]] int z_end = 0;
    __shared__ int s_range[2 * NW];
    // the flags of this wavefront's tiles, two per tile, kept in LDS when they fit (up to 32768 keys): a flag is on
    // the path of every tile, and a global load there costs a memory latency per tile
    constexpr int FLAG_TILES = 512;
    __shared__ __attribute__((aligned(16))) uint8_t s_flags[DENSE ? NW * 2 * FLAG_TILES : 4];
    __shared__ __attribute__((aligned(1024))) char s_mzone[STAGED ? NW * 2 * 4096 : 16];
    __shared__ __attribute__((aligned(1024))) char s_zero[STAGED ? 4096 : 16];      // zeros: what a tile of two all-zero blocks reads instead of a copy
    [[maybe_unused]] bool wave_done = false;      // DENSE: this wavefront's rows were computed by the launch before (it keeps the barriers company)
    if ((DENSE || LIMS) && p.mask_lims != nullptr) {
        // does every row of the block of lims_rows rows around this workgroup's have a limit?  (uniform over the workgroup)
        const int32_t* lims = mask_lims_of(p, b, hq);
        if (LIMS) {
            // (the block is this workgroup's: one row per lane, and one exchange through LDS says both whether every row has a
            // limit and what the largest is) this lane's limit, the smallest and largest of the wavefront, the largest of the workgroup
            const bool row_here = my_i < rows_b;
            const int lm = lims[p.m_si ? min(my_i, Sq - 1) : 0];
            const bool wave_ok = __builtin_amdgcn_ballot_w64(row_here && lm < 0) == 0;
            lim_lane = row_here ? min(lim_lane, lm) : 0;
            int lo = row_here ? lim_lane : 0x7fffffff, hi = lim_lane;
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) {
                lo = min(lo, __shfl_xor(lo, off, 64));
                hi = max(hi, __shfl_xor(hi, off, 64));
            }
            lim_wave_min = __builtin_amdgcn_readfirstlane(lo == 0x7fffffff ? 0 : lo);
            lim_wave_max = __builtin_amdgcn_readfirstlane(hi);
            if (lane == 0) { s_range[wave] = wave_ok ? 1 : 0; s_range[NW + wave] = lim_wave_max; }
            __syncthreads();
            bool all = true;
            int je = 0;
#pragma unroll
            for (int w2 = 0; w2 < NW; ++w2) { all = all && s_range[w2] != 0; je = max(je, s_range[NW + w2]); }
            if (__builtin_amdgcn_readfirstlane(all ? 1 : 0) == 0) return;      // the dense-mask launch computes this block
            j_end = __builtin_amdgcn_readfirstlane(je);
            n_tiles = (j_end + PF_BN - 1) / PF_BN;
        } else if (p.lims_rows >= BM) {
            const int blk0 = (q0 / p.lims_rows) * p.lims_rows, blk1 = min(blk0 + p.lims_rows, rows_b);
            bool ok = true;
            for (int i = blk0 + tid; i < blk1; i += 64 * NW) ok = ok && lims[p.m_si ? i : 0] >= 0;
            const bool wave_ok = __builtin_amdgcn_ballot_w64(!ok) == 0;
            if (lane == 0) s_range[wave] = wave_ok ? 1 : 0;
            __syncthreads();
            bool all = true;
#pragma unroll
            for (int w2 = 0; w2 < NW; ++w2) all = all && s_range[w2] != 0;
            if (__builtin_amdgcn_readfirstlane(all ? 1 : 0) != 0) return;      // the launch before this one computed the block from its limits
            __syncthreads();                                                   // (s_range is used again below)
        } else {
            // blocks of 128 rows under a workgroup of 256: the launch before computed those of them whose rows all have a limit
            const bool ok = my_i >= rows_b || lims[p.m_si ? my_i : 0] >= 0;
            const bool wave_ok = __builtin_amdgcn_ballot_w64(!ok) == 0;
            if (lane == 0) s_range[wave] = wave_ok ? 1 : 0;
            __syncthreads();
            bool all = true, mine_ok = true;
#pragma unroll
            for (int w2 = 0; w2 < NW; ++w2) {
                all = all && s_range[w2] != 0;
                if (w2 / 4 == wave / 4) mine_ok = mine_ok && s_range[w2] != 0;
            }
            if (__builtin_amdgcn_readfirstlane(all ? 1 : 0) != 0) return;
            wave_done = __builtin_amdgcn_readfirstlane(mine_ok ? 1 : 0) != 0;
            if (wave_done) lim_wave_min = lim_wave_max = 0;
            __syncthreads();
        }
    }
    const bool flags_in_lds = DENSE && n_tiles <= FLAG_TILES;
    if (DENSE) {
        mflags = mask_flags_of(p, b, hq) + (int64_t)((q0 >> 5) + wave) * nkb32;
        mrow = (const T*)p.mask + (int64_t)b * p.m_sb + (int64_t)hq * p.m_sh + (int64_t)min(my_i, Sq - 1) * p.m_si;
        int lo = 0x7fffffff, hi = -1;
        if (q0 + wave * 32 < rows_b && !wave_done)
            for (int t = lane; t < n_tiles; t += 64) {
                const int f0 = mflags[2 * t], f1 = 2 * t + 1 < nkb32 ? mflags[2 * t + 1] : 2;
                if (f0 != 2 || f1 != 2) { lo = min(lo, t); hi = max(hi, t); }
                if (flags_in_lds) { s_flags[(wave * FLAG_TILES + t) * 2] = (uint8_t)f0; s_flags[(wave * FLAG_TILES + t) * 2 + 1] = (uint8_t)f1; }
            }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            lo = min(lo, __shfl_xor(lo, off, 64));
            hi = max(hi, __shfl_xor(hi, off, 64));
        }
        w_first = __builtin_amdgcn_readfirstlane(lo);
        w_last = __builtin_amdgcn_readfirstlane(hi);
        if (lane == 0) { s_range[wave] = lo; s_range[NW + wave] = hi; }
        if (STAGED && tid < 256) *(uint4v*)(s_zero + tid * 16) = uint4v{0u, 0u, 0u, 0u};
        __syncthreads();
        int g_lo = s_range[0], g_hi = s_range[NW];
#pragma unroll
        for (int w2 = 1; w2 < NW; ++w2) { g_lo = min(g_lo, s_range[w2]); g_hi = max(g_hi, s_range[NW + w2]); }
        // (uniform by construction; said explicitly, because tile numbers end up in scalar DMA descriptors)
        t_first = __builtin_amdgcn_readfirstlane(g_hi < 0 ? 0 : g_lo);
        n_tiles = __builtin_amdgcn_readfirstlane(g_hi + 1);      // (0 when the mask hides everything from these 128 rows)
        // z_end: the first tile after t_first in which the mask does something to this wavefront's rows; the tiles
        // t_first + 1 .. z_end - 1 run through the pipelined loop like tiles of a launch without a mask.  (STAGED: the first
        // tile that the mask hides from this wavefront altogether, which it skips - every other tile has its values in LDS,
        // zeros and -inf included, and goes through the pipelined loop)
        int z = n_tiles;
        for (int t = t_first + 1 + lane; t < n_tiles; t += 64) {
            const int f0 = mflags[2 * t], f1 = 2 * t + 1 < nkb32 ? mflags[2 * t + 1] : 2;
            if (STAGED ? (f0 == 2 && f1 == 2) : (f0 != 1 || f1 != 1)) { z = t; break; }
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) z = min(z, __shfl_xor(z, off, 64));
        z_end = __builtin_amdgcn_readfirstlane(z);
    }

    // flag of 32-key block blk (= 2 * tile + half) for this wavefront's rows; past the last block: hidden
    [[maybe_unused]] auto flag_of = [&](int blk) __attribute__((always_inline)) -> int {
        if (blk >= nkb32) return 2;
        const int f = flags_in_lds ? (int)s_flags[wave * FLAG_TILES * 2 + blk] : (int)mflags[blk];
        return __builtin_amdgcn_readfirstlane(f);
    };
    // both flags of tile t in one value: the second block's in bits 8 - 15 (one LDS read where the flags are there: this sits
    // in front of every tile's copies and in every pipelined iteration)
    [[maybe_unused]] auto tile_flags = [&](int t) __attribute__((always_inline)) -> unsigned {
        unsigned f2;
        if (flags_in_lds) f2 = *(const unsigned short*)&s_flags[(wave * FLAG_TILES + t) * 2];
        else f2 = (unsigned)flag_of(2 * t) | ((unsigned)flag_of(2 * t + 1) << 8);
        return (unsigned)__builtin_amdgcn_readfirstlane((int)f2);
    };
    // STAGED: the copies of this wavefront's 32 rows x 64 keys of the mask for tile t into its buffer t % 2.  Copy c, lane l:
    // row 8 c + l / 8, position l % 8 of the row's eight 16-byte chunks, which takes chunk (l % 8) ^ ((row / 2) % 8).  The
    // descriptor starts at the wavefront's first row and ends with the head's last row (rows past Sq deliver zeros).
    // ((row / 2) % 8 = (l / 16) ^ 4 (c % 2): two lane offsets serve the four copies, the rows' 8 c go into the scalar offset)
    [[maybe_unused]] int m_voff[2];
    [[maybe_unused]] int m_rd = 0;                 // this lane's read position in a buffer, before the XOR with the chunk it wants
    [[maybe_unused]] uint4v m_desc = {0u, 0u, 0u, 0u};
    [[maybe_unused]] unsigned m_lds = 0;
    if (STAGED) {
        const int row0 = q0 + wave * 32;
#pragma unroll
        for (int c = 0; c < 2; ++c) m_voff[c] = (int)((int64_t)(lane >> 3) * p.m_si * 2) + (((lane & 7) ^ (lane >> 4) ^ (4 * c)) << 4);
        m_rd = ql * 128 + g * 8 + (((ql >> 1) & 7) << 4);
        const int64_t left = row0 < Sq ? ((int64_t)(Sq - 1 - row0) * p.m_si + Skv) * 2 : 0;
        m_desc = dma_descriptor((const T*)p.mask + (int64_t)b * p.m_sb + (int64_t)hq * p.m_sh + (int64_t)row0 * p.m_si,
                                (int)(left > 0x7fffffffLL ? 0x7fffffffLL : left));
        m_lds = lds_address(s_mzone) + wave * 2 * 4096;
    }
    [[maybe_unused]] auto issue_m = [&](int t) __attribute__((always_inline)) {
        if (t >= n_tiles) return;
        // not for a tile the mask hides from this wavefront altogether (it skips the tile), nor for one of two all-zero blocks
        // (it reads the zeros of s_zero instead)
        if (tile_flags(t) == 0x0202u || tile_flags(t) == 0x0101u) return;
#pragma unroll
        for (int c = 0; c < 4; ++c) dma_copy16_at(m_desc, m_lds + (t & 1) * 4096 + c * 1024, m_voff[c % 2], t * PF_BN * 2 + c * 8 * (int)p.m_si * 2);
    };

    // ---- global -> LDS copy plan ---------------------------------------------------
    // wavefront-wide load number ii = wave*LPW + c fills LDS bytes [ii*1024, ii*1024 + 1024)
    // of a tile; lane -> position p = ii*64 + lane -> (row, slot) -> global chunk slot ^ f(row).
    int k_voff[LPW], v_voff[LPW];
#pragma unroll
    for (int c = 0; c < LPW; ++c) {
        const int pos = (wave * LPW + c) * 64 + lane;
        const int row = pos / L::CPR, slot = pos % L::CPR;
        k_voff[c] = dma_chunk_offset(row, (int)p.k_ss * 2, slot ^ L::fk(row), p.D * 2);
        v_voff[c] = dma_chunk_offset(row, (int)p.v_ss * 2, slot ^ L::fv(row), p.Dv * 2);
    }
    const int64_t k_tile_bytes = (int64_t)PF_BN * p.k_ss * 2, v_tile_bytes = (int64_t)PF_BN * p.v_ss * 2;
    // K buffer b at smem + b*TILE, V buffer b at smem + (2+b)*TILE.  Tiles are copied in order from tile t_first on, so
    // the copy state runs along: address of the next tile and the bytes from there to the end of the last row this
    // workgroup may see (loads past that return 0; rows past a batch entry's key count are never read).
    const char* k_next = (const char*)kp + t_first * k_tile_bytes;
    const char* v_next = (const char*)vp + t_first * v_tile_bytes;
    int64_t k_rem = (int64_t)(j_end - t_first * PF_BN - 1) * p.k_ss * 2 + p.D * 2;
    int64_t v_rem = (int64_t)(j_end - t_first * PF_BN - 1) * p.v_ss * 2 + p.Dv * 2;
    auto clamp31 = [](int64_t x) __attribute__((always_inline)) {
        const unsigned hi = (unsigned)((unsigned long long)x >> 32), lo = (unsigned)x;
        return (hi | (lo >> 31)) != 0 ? 0x7fffffff : (int)lo;
    };
    auto issue_k = [&](int /*t: the next tile in order*/, int buf) __attribute__((always_inline)) {
        const uint4v r = dma_descriptor(k_next, clamp31(k_rem));
        const unsigned dst = lds_address(smem) + buf * L::TILE_BYTES + wave * LPW * 1024;
#pragma unroll
        for (int c = 0; c < LPW; ++c) dma_copy16(r, dst + c * 1024, k_voff[c]);
        k_next += k_tile_bytes;
        k_rem -= k_tile_bytes;
    };
    auto issue_v = [&](int, int buf) __attribute__((always_inline)) {
        const uint4v r = dma_descriptor(v_next, clamp31(v_rem));
        const unsigned dst = lds_address(smem) + (2 + buf) * L::TILE_BYTES + wave * LPW * 1024;
#pragma unroll
        for (int c = 0; c < LPW; ++c) dma_copy16(r, dst + c * 1024, v_voff[c]);
        v_next += v_tile_bytes;
        v_rem -= v_tile_bytes;
    };

    // The Q rows are asked for first (fetch_q_rows: 16 bytes per lane, eight lanes to a run of a row); they reach the operand
    // layout through LDS below.
    constexpr int NQH = D / 64;      // passes of 64 columns
    uint4v qraw[NQH][4];
    fetch_q_rows(qraw, qp, q0 + wave * 32, Sq, p.q_ss, p.D, lane);
    // The first copies start before anything waits on memory: K of the first two tiles.  V of the first tile follows after
    // the barrier below: until then the V buffers are the staging area of the Q rows.
    if (n_tiles > t_first) {
        issue_k(t_first, t_first & 1);
        if (t_first + 1 < n_tiles) issue_k(t_first + 1, (t_first + 1) & 1);
        if (STAGED) { issue_m(t_first); issue_m(t_first + 1); }
    }

    // ---- LDS read addresses (bytes inside a tile buffer) ------------------------------------
    // K operand: lane (ql, g) reads row 32*kb + ql, logical chunk 2*s + g
    int k_addr[NSTEP];
    {
        const int F = L::fk(ql);
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) k_addr[s] = ql * L::ROWB + (((2 * s + g) ^ F) << 4);
    }
    // V operand (transposing read): the 16 lanes of a group fetch a 4-key x 16-d patch
    // (lane n: key n/4, d 4*(n%4)..+3) and receive (d = n, keys 0..3).  Row within a
    // 16-row block: 8*h + 4*g + n/4; logical chunk 4*db + 2*dh + (n%4)/2.
    int v_addr[NDB][2];
    {
        const int n = lane & 15, dh = (lane >> 4) & 1;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int r = 8 * h + 4 * g + (n >> 2);
                const int chunk = 4 * db + 2 * dh + ((n & 3) >> 1);
                v_addr[db][h] = r * L::ROWB + ((chunk ^ L::fv(r)) << 4) + (n & 1) * 8;
            }
    }

    // ---- Q^T operand, resident in registers ---------------------------------------
    // through this wavefront's 4 KiB of the V buffers, which nothing is copied into before the barrier below
    vec8 qreg[NSTEP];
    static_assert(2 * L::TILE_BYTES >= NW * 4096, "the K buffers, and the V buffers, hold a 4 KiB staging area per wavefront");
    stage_q_rows(qreg, qraw, smem + 2 * L::TILE_BYTES + wave * 4096, lane);
    // Fold scale * log2(e) into Q once (rounded back to the storage type): the matrix product then
    // yields the scores directly in the log2 units the softmax works in.
    const float c2 = p.scale * 1.4426950408889634f;
#pragma unroll
    for (int s = 0; s < NSTEP; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) qreg[s][e] = (T)((float)qreg[s][e] * c2);

    floatx16 o_acc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[db][r] = 0.0f;
    // Reference maximum m_ref (log2 units) of this lane's query.  It is baked into the matrix product:
    // the first MFMA of every score block starts from the accumulator neg_ref = -m_ref instead of 0, so
    // the product delivers s - m_ref and the probabilities are a bare exp2 of it.  m_ref is set from the
    // first tile that holds a visible key and afterwards only raised, when a tile maximum exceeds it by
    // more than 2^8 (lazy rescaling: exact in exact arithmetic, probabilities stay <= 2^8).
    float m_ref = 0.0f;
    bool inited = false;
    floatx16 neg_ref;
#pragma unroll
    for (int r = 0; r < 16; ++r) neg_ref[r] = 0.0f;
    float l_run = 0.0f;           // this lane's share of the running denominator

    // ---- matrix operands in flight ---------------------------------------------------------------
    constexpr int KD = PF_KD < NSTEP ? PF_KD : NSTEP;   // K operands are fetched KD k-steps (2*KD MFMAs) ahead
    constexpr int NPV = 4 * NDB;                   // MFMAs of one O^T update (4 k-steps of 16 keys x NDB blocks)
    constexpr int VD = PF_VD;                      // V operands are fetched VD MFMAs ahead
    vec8 kbuf[KD][2];
    vec8 vbuf[VD];
    auto read_k = [&](const char* kb, int s) __attribute__((always_inline)) {
#pragma unroll
        for (int b2 = 0; b2 < 2; ++b2) kbuf[s % KD][b2] = *(const vec8*)(kb + k_addr[s] + b2 * 32 * L::ROWB);
    };
    auto read_v = [&](const char* vb, int i) __attribute__((always_inline)) {      // i = ks * NDB + db
        const int ks = i / NDB, db = i % NDB;
        short8v av;
        av.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (short4v __attribute__((address_space(3)))*)(vb + v_addr[db][0] + ks * 16 * L::ROWB));
        av.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (short4v __attribute__((address_space(3)))*)(vb + v_addr[db][1] + ks * 16 * L::ROWB));
        vbuf[i % VD] = __builtin_bit_cast(vec8, av);
    };

    // Two score tiles are alive at a time: S(t) is turned into probabilities while the matrix pipe
    // already computes S(t+1).  sacc[t % 2] holds S(t) - m_ref.
    floatx16 sacc[2][2];
    vec8 pb[4];
    float tmax = -INFINITY;       // maximum of the current score tile relative to m_ref (both halves of the query's lanes)
    float rsum = 0.0f;

    // register r of block kb of a score tile that starts at key j0 is key j0 + 32*kb + 8*(r/4) + 4*g + (r%4)
    auto mask_tile = [&](floatx16 (&sx)[2], int j0) __attribute__((always_inline)) {
        const int rel = lim_lane - (j0 + 4 * g);
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int kofs = 32 * kb + 8 * (r / 4) + (r % 4);
                if (kofs >= rel) sx[kb][r] = -INFINITY;
            }
    };
    // Move the reference maximum when the pending tile maximum asks for it (first visible tile, or more
    // than the threshold above the reference): rescales what has been accumulated and the pending tile.
    auto adjust_reference = [&](floatx16 (&sx)[2]) __attribute__((always_inline)) {
        const bool need = inited ? (tmax > PF_RESCALE_THRESHOLD - SHIFT) : (tmax > -INFINITY);
        if (__builtin_amdgcn_ballot_w64(need) != 0) {
            const float delta = need ? tmax + SHIFT : 0.0f;       // lanes that do not need it move by 0
            tmax -= delta;
            const float alpha = inited ? __builtin_amdgcn_exp2f(-delta) : 1.0f;   // nothing accumulated yet: nothing to rescale
            m_ref += delta;
            inited = inited || need;
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) o_acc[db][r] *= alpha;
#pragma unroll
            for (int r = 0; r < 16; ++r) neg_ref[r] = -m_ref;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) sx[kb][r] -= delta;
        }
    };
    // Probabilities of 4 score registers (slice sl = 0..7 of a tile): P^T in storage precision; element e of
    // k-step ks is register 8*(ks%2)+e of key block ks/2, i.e. key 16*ks + 8*(e/4) + 4*g + (e%4).  The
    // denominator is summed from the rounded values, two per instruction (dot2 with ones, f32 accumulate).
    auto softmax_slice = [&](floatx16 (&sx)[2], int sl) __attribute__((always_inline)) {
        const int ks = sl / 2, e0 = 4 * (sl % 2);
#pragma unroll
        for (int e = e0; e < e0 + 4; ++e) pb[ks][e] = (T)__builtin_amdgcn_exp2f(sx[ks / 2][8 * (ks % 2) + e]);
#pragma unroll
        for (int e = e0; e < e0 + 4; e += 2) {
            typename Mma<T>::vec2 pr = {pb[ks][e], pb[ks][e + 1]};
            rsum = Mma<T>::add2(pr, rsum);
        }
    };
    auto max_of = [&](floatx16 (&sx)[2]) __attribute__((always_inline)) {
        float m = sx[0][0];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) m = fmaxf(m, sx[kb][r]);
        return xor32_max(m);
    };

#define SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
    constexpr int SG_MFMA = 0x8, SG_VALU = 0x2, SG_TRANS = 0x400, SG_DSR = 0x100;

    // start of every iteration t: K(t+1) and V(t) are in LDS for everyone, everyone is past S^T(t) (K buffer
    // t%2 is free) and past O^T(t-1) (V buffer (t+1)%2 is free); start the next global loads into those.
    auto turn_sync = [&]() __attribute__((always_inline)) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    };
    auto turn_issue = [&](int t) __attribute__((always_inline)) {
        if (STAGED) issue_m(t + 2);      // (into the buffer of tile t, whose values were taken before this turn; first: it reads a flag)
        if (t + 2 < n_tiles) issue_k(t + 2, t & 1);
        if (t + 1 < n_tiles) issue_v(t + 1, (t + 1) & 1);
    };
    auto turn = [&](int t) __attribute__((always_inline)) {
        turn_sync();
        turn_issue(t);
    };

    // Hot iteration (tiles t and t+1 both computed by this wavefront, tile t+1 needs no mask):
    // probabilities of tile t (scores in sacc[par], their maximum in tmax) on the vector ALU while the matrix
    // pipe computes the scores of tile t+1; then O^T += V(t)^T P(t)^T with the maximum of S^T(t+1) underneath.
    // WITH_M (STAGED): the mask's 32 values for this lane's scores of tile t + 1 are taken from the wavefront's buffer (zeros,
    // -inf and values alike) and added on the way into the maximum, under the matrix instructions of the O^T update.
    auto iter = [&](int t, auto PAR_, auto WITH_M_) __attribute__((always_inline)) {
        constexpr int par = decltype(PAR_)::value;
        constexpr bool WITH_M = decltype(WITH_M_)::value;
        floatx16 (&sc)[2] = sacc[par];
        floatx16 (&sn)[2] = sacc[1 - par];
        const char* k_nxt = smem + (1 - par) * L::TILE_BYTES;        // K(t+1)
        const char* v_cur = smem + (2 + par) * L::TILE_BYTES;        // V(t)
        turn_sync();
#pragma unroll
        for (int s = 0; s < KD; ++s) read_k(k_nxt, s);
        turn_issue(t);
        adjust_reference(sc);
        rsum = 0.0f;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
#pragma unroll
            for (int b2 = 0; b2 < 2; ++b2)
                sn[b2] = Mma<T>::run(kbuf[s % KD][b2], qreg[s], s == 0 ? neg_ref : sn[b2]);
            if (s + KD < NSTEP) read_k(k_nxt, s + KD);
#pragma unroll
            for (int sl = slice_lo(s); sl < slice_lo(s + 1); ++sl) softmax_slice(sc, sl);
            if (s >= NSTEP - VD / 2) { read_v(v_cur, 2 * (s - (NSTEP - VD / 2))); read_v(v_cur, 2 * (s - (NSTEP - VD / 2)) + 1); }
        }
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                SGB(SG_MFMA, 1);
                if (slice_lo(s + 1) - slice_lo(s) == 1) { SGB(SG_TRANS, 2); SGB(SG_VALU, 2); } else { SGB(SG_TRANS, 4); SGB(SG_VALU, 4); }
                if (s + KD < NSTEP) SGB(SG_DSR, 1);
                if (s >= NSTEP - VD / 2) SGB(SG_DSR, 2);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        l_run += rsum;
        float m0 = WITH_M ? -INFINITY : sn[0][0], m1 = WITH_M ? -INFINITY : sn[1][0];
        typedef T vec4 __attribute__((ext_vector_type(4)));
        [[maybe_unused]] vec4 mv[2][2];      // the values of registers 4 r4 .. 4 r4 + 3 of both key blocks, read one group of four ahead
        [[maybe_unused]] const char* mz = s_mzone + (wave * 2 + 1 - par) * 4096;      // (t + 1 has the parity 1 - par)
        if (WITH_M && tile_flags(t + 1) == 0x0101u) mz = s_zero;
        [[maybe_unused]] auto read_m = [&](int r4) __attribute__((always_inline)) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) mv[r4 % 2][kb] = *(const vec4*)(mz + (m_rd ^ ((4 * kb + r4) << 4)));
        };
        if (WITH_M) read_m(0);
#pragma unroll
        for (int i = 0; i < NPV; ++i) {
            o_acc[i % NDB] = Mma<T>::run(vbuf[i % VD], pb[i / NDB], o_acc[i % NDB]);
            if (i + VD < NPV) read_v(v_cur, i + VD);
#pragma unroll
            for (int r = pair_lo(i); r < pair_lo(i + 1); ++r) {
                if (WITH_M) {
                    if (r % 4 == 0 && r + 4 < 16) read_m(r / 4 + 1);
                    sn[0][r] = __builtin_fmaf((float)mv[(r / 4) % 2][0][r % 4], 1.4426950408889634f, sn[0][r]);
                    sn[1][r] = __builtin_fmaf((float)mv[(r / 4) % 2][1][r % 4], 1.4426950408889634f, sn[1][r]);
                }
                m0 = fmaxf(m0, sn[0][r]);
                m1 = fmaxf(m1, sn[1][r]);
            }
        }
        tmax = xor32_max(fmaxf(m0, m1));
    };

    // The same iteration with the cheap overflow check (ORCHK): no maxima.  The probabilities of tile t are OR-ed
    // together as they are packed; a set bit 14 in either half of the result says that one of them reached 2, i.e. that
    // a score of tile t passed the reference by more than 2^SHIFT.  Only then (rare: the reference is the maximum of
    // an earlier tile) the exact path runs: maximum of tile t, reference moved, O^T and the row sum rescaled, both score
    // tiles shifted and the probabilities of tile t taken again - before anything of tile t has been accumulated.
    // (WITH_M as in iter: the mask's values for tile t + 1 go onto its scores under the O^T update; the check of the next
    // iteration then sees probabilities of scores that carry them)
    auto iter_or = [&](int t, auto PAR_, auto WITH_M_) __attribute__((always_inline)) {
        constexpr int par = decltype(PAR_)::value;
        constexpr bool WITH_M = decltype(WITH_M_)::value;
        floatx16 (&sc)[2] = sacc[par];
        floatx16 (&sn)[2] = sacc[1 - par];
        const char* k_nxt = smem + (1 - par) * L::TILE_BYTES;        // K(t+1)
        const char* v_cur = smem + (2 + par) * L::TILE_BYTES;        // V(t)
        turn_sync();
#pragma unroll
        for (int s = 0; s < KD; ++s) read_k(k_nxt, s);
        turn_issue(t);
        unsigned orv = 0;
        // exponentials of slice sl (4 scores) now, their packing one slice later: a pack never waits for its operands
        float ex[2][4];
        typedef unsigned uint4w __attribute__((ext_vector_type(4)));
        auto exps_of = [&](int sl) __attribute__((always_inline)) {
            const int ks = sl / 2, e0 = 4 * (sl % 2);
#pragma unroll
            for (int e = 0; e < 4; ++e) ex[sl % 2][e] = __builtin_amdgcn_exp2f(sc[ks / 2][8 * (ks % 2) + e0 + e]);
        };
        auto pack_of = [&](int sl) __attribute__((always_inline)) {
            const int ks = sl / 2, e0 = 4 * (sl % 2);
#pragma unroll
            for (int e = 0; e < 4; ++e) pb[ks][e0 + e] = (T)ex[sl % 2][e];
            const uint4w w = __builtin_bit_cast(uint4w, pb[ks]);
            orv = orv | w[e0 / 2] | w[e0 / 2 + 1];
        };
        constexpr int NSL = 8;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
#pragma unroll
            for (int b2 = 0; b2 < 2; ++b2)
                sn[b2] = Mma<T>::run(kbuf[s % KD][b2], qreg[s], s == 0 ? neg_ref : sn[b2]);
            if (s + KD < NSTEP) read_k(k_nxt, s + KD);
#pragma unroll
            for (int sl = slice_lo(s); sl < slice_lo(s + 1); ++sl) {
                exps_of(sl);
                if (sl > 0) pack_of(sl - 1);
            }
            if (s >= NSTEP - VD / 2) { read_v(v_cur, 2 * (s - (NSTEP - VD / 2))); read_v(v_cur, 2 * (s - (NSTEP - VD / 2)) + 1); }
        }
        pack_of(NSL - 1);
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                SGB(SG_MFMA, 1);
                if (slice_lo(s + 1) - slice_lo(s) == 1) {
                    SGB(SG_TRANS, 1);
                    if (s > 0) SGB(SG_VALU, 1);
                    SGB(SG_TRANS, 1);
                    if (s > 0 && h == 1) SGB(SG_VALU, 1);
                } else {
                    SGB(SG_TRANS, 2); SGB(SG_VALU, 2); SGB(SG_TRANS, 2); SGB(SG_VALU, 1);
                }
                if (s + KD < NSTEP) SGB(SG_DSR, 1);
                if (s >= NSTEP - VD / 2) SGB(SG_DSR, 2);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (__builtin_amdgcn_ballot_w64((orv & 0x40004000u) != 0) != 0) {
            tmax = max_of(sc);
            const bool need = tmax > PF_RESCALE_THRESHOLD - SHIFT;
            const float delta = need ? tmax + SHIFT : 0.0f;
            const float alpha = __builtin_amdgcn_exp2f(-delta);
            m_ref += delta;
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) o_acc[db][r] *= alpha;
#pragma unroll
            for (int r = 0; r < 16; ++r) neg_ref[r] = -m_ref;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) { sc[kb][r] -= delta; sn[kb][r] -= delta; }
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                for (int e = 0; e < 8; ++e) pb[ks][e] = (T)__builtin_amdgcn_exp2f(sc[ks / 2][8 * (ks % 2) + e]);
        }
        __builtin_amdgcn_sched_barrier(0);
        float rs[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        typedef T vec4 __attribute__((ext_vector_type(4)));
        [[maybe_unused]] vec4 mv[2][2];      // the values of registers 4 r4 .. 4 r4 + 3 of both key blocks, read one group of four ahead
        [[maybe_unused]] const char* mz = s_mzone + (wave * 2 + 1 - par) * 4096;      // (t + 1 has the parity 1 - par)
        if (WITH_M && tile_flags(t + 1) == 0x0101u) mz = s_zero;
        [[maybe_unused]] auto read_m = [&](int r4) __attribute__((always_inline)) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) mv[r4 % 2][kb] = *(const vec4*)(mz + (m_rd ^ ((4 * kb + r4) << 4)));
        };
        if (WITH_M) read_m(0);
#pragma unroll
        for (int i = 0; i < NPV; ++i) {
            o_acc[i % NDB] = Mma<T>::run(vbuf[i % VD], pb[i / NDB], o_acc[i % NDB]);
            if (i + VD < NPV) read_v(v_cur, i + VD);
            // row sum of the rounded probabilities, two per instruction, four chains
#pragma unroll
            for (int ii = pair_lo(i); ii < pair_lo(i + 1); ++ii) {
                typename Mma<T>::vec2 pr = {pb[ii / 4][2 * (ii % 4)], pb[ii / 4][2 * (ii % 4) + 1]};
                rs[ii % 4] = Mma<T>::add2(pr, rs[ii % 4]);
                if (WITH_M) {
                    const int r = ii;
                    if (r % 4 == 0 && r + 4 < 16) read_m(r / 4 + 1);
                    sn[0][r] = __builtin_fmaf((float)mv[(r / 4) % 2][0][r % 4], 1.4426950408889634f, sn[0][r]);
                    sn[1][r] = __builtin_fmaf((float)mv[(r / 4) % 2][1][r % 4], 1.4426950408889634f, sn[1][r]);
                }
            }
        }
        if (!WITH_M) {
#pragma unroll
            for (int i = 0; i < NPV; ++i) {
                SGB(SG_MFMA, 1);
                if (pair_lo(i + 1) - pair_lo(i) == 1) SGB(SG_VALU, 1); else SGB(SG_VALU, 2);
                if (i + VD < NPV) SGB(SG_DSR, 2);
            }
        }
        asm volatile("" : "+v"(rs[0]), "+v"(rs[1]), "+v"(rs[2]), "+v"(rs[3]));      // (keeps the sums from being sunk below the next barrier)
        __builtin_amdgcn_sched_barrier(0);
        rsum = (rs[0] + rs[1]) + (rs[2] + rs[3]);
        l_run += rsum;
    };

    // Dense mask on the scores of the tile that starts at key j0 (scores are in log2 units): per 32-key half, nothing
    // where the flag says zeros, -inf where it says hidden, else the values themselves - 4 consecutive keys per load
    // where the mask's layout allows (unit key stride, 8-byte aligned rows), element by element otherwise.
    auto add_dense_mask = [&](floatx16 (&sx)[2], int j0) __attribute__((always_inline)) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            const int flag = flag_of((j0 >> 5) + kb);
            if (flag == 1) continue;
            if (flag == 2) {
#pragma unroll
                for (int r = 0; r < 16; ++r) sx[kb][r] = -INFINITY;
                continue;
            }
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const int j = j0 + 32 * kb + 8 * r4 + 4 * g;
                typedef T vec4 __attribute__((ext_vector_type(4)));
                vec4 mv;
                if (STAGED) mv = *(const vec4*)(s_mzone + (wave * 2 + ((j0 / PF_BN) & 1)) * 4096 + (m_rd ^ ((4 * kb + r4) << 4)));
                else if (p.mask_vec && j + 3 < Skv) mv = *(const vec4*)(mrow + j);
                else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) mv[e] = mrow[(int64_t)min(j + e, Skv - 1) * p.m_sj];
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) sx[kb][4 * r4 + e] = __builtin_fmaf((float)mv[e], 1.4426950408889634f, sx[kb][4 * r4 + e]);
            }
        }
    };
    // scores of one tile without overlap (prologue and the last tiles of a wavefront); kb = K tile in LDS
    auto scores_plain = [&](const char* kb, floatx16 (&sx)[2], int j0) __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < KD; ++s) read_k(kb, s);
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
#pragma unroll
            for (int b2 = 0; b2 < 2; ++b2) sx[b2] = Mma<T>::run(kbuf[s % KD][b2], qreg[s], s == 0 ? neg_ref : sx[b2]);
            if (s + KD < NSTEP) read_k(kb, s + KD);
        }
        if (DENSE) add_dense_mask(sx, j0);
        if (j0 + PF_BN > lim_wave_min) mask_tile(sx, j0);
        tmax = max_of(sx);
    };

    // tiles this wavefront computes, and how many of them the hot loop may produce scores for
    const int n_act = lim_wave_max > 0 ? (lim_wave_max + PF_BN - 1) / PF_BN : 0;
    const int n_hot = lim_wave_min > 0 ? min(lim_wave_min / PF_BN, n_act) : 0;      // tiles 0..n_hot-1 need no mask

    if (!DENSE && n_tiles > t_first) {
        // prologue: K and V of the first tile (tile 0, or a split's first: an even one) and K of the next are in flight since
        // the start; scores of the first tile
        __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0), told to the compiler too: it then knows the Q rows have arrived
        asm volatile("" ::: "memory");
        __syncthreads();
        issue_v(t_first, t_first & 1);           // (every wavefront has its Q rows out of the V buffers)
        if (n_act > t_first) scores_plain(smem, sacc[0], t_first * PF_BN);
        int t = t_first;
        if constexpr (ORCHK) {
            if (t_first + 2 < n_hot) {
                // the reference of every row of this wavefront: the maximum of the first tile (nothing accumulated yet,
                // so nothing to rescale)
                {
                    const bool need = tmax > -INFINITY;
                    const float delta = need ? tmax + SHIFT : 0.0f;
                    m_ref += delta;
                    tmax -= delta;
                    inited = inited || need;
#pragma unroll
                    for (int r = 0; r < 16; ++r) neg_ref[r] = -m_ref;
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                        for (int r = 0; r < 16; ++r) sacc[0][kb][r] -= delta;
                }
                for (; t + 2 < n_hot; t += 2) {
                    iter_or(t, std::integral_constant<int, 0>{}, std::integral_constant<bool, STAGED>{});
                    iter_or(t + 1, std::integral_constant<int, 1>{}, std::integral_constant<bool, STAGED>{});
                }
                tmax = max_of(sacc[0]);           // the masked loop below decides by maxima
            }
        } else {
            for (; t + 2 < n_hot; t += 2) {
                iter(t, std::integral_constant<int, 0>{}, std::false_type{});
                iter(t + 1, std::integral_constant<int, 1>{}, std::false_type{});
            }
        }
        // the rest, one tile at a time without overlap; the pending scores are in sacc[0]
        for (; t < n_tiles; ++t) {
            turn(t);
            if (t < n_act) {
                const char* v_cur = smem + (2 + (t & 1)) * L::TILE_BYTES;
#pragma unroll
                for (int i = 0; i < VD; ++i) read_v(v_cur, i);
                adjust_reference(sacc[0]);
                rsum = 0.0f;
#pragma unroll
                for (int sl = 0; sl < 8; ++sl) softmax_slice(sacc[0], sl);
                l_run += rsum;
#pragma unroll
                for (int i = 0; i < NPV; ++i) {
                    o_acc[i % NDB] = Mma<T>::run(vbuf[i % VD], pb[i / NDB], o_acc[i % NDB]);
                    if (i + VD < NPV) read_v(v_cur, i + VD);
                }
                if (t + 1 < n_act) scores_plain(smem + ((t + 1) & 1) * L::TILE_BYTES, sacc[0], (t + 1) * PF_BN);
            }
        }
    }
    if (DENSE && n_tiles > t_first) {
        // The same one-tile-at-a-time loop over the tiles t_first .. n_tiles - 1 the mask leaves to this workgroup; a
        // wavefront computes tile t if its limits (causal, key count) and the mask's flags leave it a visible block.
        auto mine = [&](int t) __attribute__((always_inline)) {
            if (t >= n_act || t < w_first || t > w_last) return false;
            return flag_of(2 * t) != 2 || flag_of(2 * t + 1) != 2;
        };
        __builtin_amdgcn_s_waitcnt(0x0F70);
        asm volatile("" ::: "memory");
        __syncthreads();
        issue_v(t_first, t_first & 1);
        bool pending = mine(t_first);
        if (pending) scores_plain(smem + (t_first & 1) * L::TILE_BYTES, sacc[0], t_first * PF_BN);
        int t = t_first;
        auto plain_step = [&]() __attribute__((always_inline)) {
            turn(t);
            if (pending) {
                const char* v_cur = smem + (2 + (t & 1)) * L::TILE_BYTES;
#pragma unroll
                for (int i = 0; i < VD; ++i) read_v(v_cur, i);
                adjust_reference(sacc[0]);
                rsum = 0.0f;
#pragma unroll
                for (int sl = 0; sl < 8; ++sl) softmax_slice(sacc[0], sl);
                l_run += rsum;
#pragma unroll
                for (int i = 0; i < NPV; ++i) {
                    o_acc[i % NDB] = Mma<T>::run(vbuf[i % VD], pb[i / NDB], o_acc[i % NDB]);
                    if (i + VD < NPV) read_v(v_cur, i + VD);
                }
            }
            pending = t + 1 < n_tiles && mine(t + 1);
            if (pending) scores_plain(smem + ((t + 1) & 1) * L::TILE_BYTES, sacc[0], (t + 1) * PF_BN);
            ++t;
        };
        // the run of tiles after the first one that neither the mask nor a limit touches: pipelined, two at a time
        // from an even tile on
        const int hot_end = min(min(z_end, n_hot), n_tiles);
        if constexpr (BF16) {
            // bf16: without maxima, as in a launch without a mask - once every row of the wavefront has a reference.  A
            // row the mask has hidden entirely so far has none; the plain iteration knows how to give it one.
            while (t < n_tiles) {
                if (pending && !(t & 1) && t + 2 < hot_end && __builtin_amdgcn_ballot_w64(!inited) == 0) {
                    adjust_reference(sacc[0]);
                    for (; t + 2 < hot_end; t += 2) {
                        iter_or(t, std::integral_constant<int, 0>{}, std::integral_constant<bool, STAGED>{});
                        iter_or(t + 1, std::integral_constant<int, 1>{}, std::integral_constant<bool, STAGED>{});
                    }
                    tmax = max_of(sacc[0]);
                }
                plain_step();
            }
        } else {
            // (STAGED: every tile's values are in LDS, zeros and -inf included, and the pipelined iteration adds them all: one code path)
            if ((t & 1) && t < n_tiles) plain_step();
            if (pending)
                for (; t + 2 < hot_end; t += 2) {
                    iter(t, std::integral_constant<int, 0>{}, std::integral_constant<bool, STAGED>{});
                    iter(t + 1, std::integral_constant<int, 1>{}, std::integral_constant<bool, STAGED>{});
                }
            while (t < n_tiles) plain_step();
        }
    }
#undef SGB

    // ---- normalise and store ------------------------------------------------------------------
    if (DENSE && wave_done) return;      // (every barrier is behind)
    const float l_tot = xor32_sum(l_run);
    if constexpr (SPLIT) {
        // partial result of this split: unnormalised O, and (reference, sum) in the log2 units the combine kernel takes for
        // 16-bit storage; a row that saw no key in this split says so with a reference of -inf
        if (my_i < rows_b) {
            const int64_t slot = (((int64_t)b * p.Hq + hq) * Sq + my_i) * p.num_splits + split;
            float* arow = p.ws_acc + slot * D + g * 4;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    typedef float f4 __attribute__((ext_vector_type(4)));
                    f4 w = {o_acc[db][r4 * 4], o_acc[db][r4 * 4 + 1], o_acc[db][r4 * 4 + 2], o_acc[db][r4 * 4 + 3]};
                    *(f4*)(arow + db * 32 + r4 * 8) = w;
                }
            if (g == 0) {
                p.ws_ml[slot * 2 + 0] = l_tot == 0.0f ? -INFINITY : m_ref;
                p.ws_ml[slot * 2 + 1] = l_tot;
            }
        }
        return;
    }
    const float inv = (l_tot == 0.0f) ? __builtin_nanf("") : 1.0f / l_tot;   // no visible key: NaN, as the reference
    if (p.lse && g == 0 && my_i < rows_b)       // m_ref and the sum are in log2 units of the scaled scores
        p.lse[((int64_t)b * p.Hq + hq) * Sq + my_i] = l_tot == 0.0f ? -INFINITY : (m_ref + __builtin_log2f(l_tot)) * 0.6931471805599453f;
    // store_o_rows through this wavefront's 4 KiB of the K buffers: nobody reads K after the barrier of the workgroup's last
    // tile (a slower wavefront may still be reading V, which lies behind them).
    store_o_rows(o_acc, inv, smem + wave * 4096, op, q0 + wave * 32, rows_b, p.o_ss, p.Dv, lane);
#endif
}

hipError_t launch_sdpa_combine(const SdpaParams& p, int dtype, hipStream_t stream);

template <typename T, int D, int MASK, int NW>
static hipError_t launch_prefill_nw(const SdpaParams& p0, hipStream_t stream)
{
    SdpaParams p = p0;
    const int nqb = (p.Sq + 32 * NW - 1) / (32 * NW);
    const int64_t total = (int64_t)nqb * p.Hq * p.B;
    // 256 registers per lane: eight wavefronts per compute unit, i.e. two workgroups of four or one of eight; an eighth
    // of the compute units per XCD
    p.interleave = work_interleave(p.causal != 0 || p.mask != nullptr, (8 / NW) * device_cus() / 8, p.G, nqb, (total & 7) == 0 ? total >> 3 : total);
    p.deal_groups = (total & 7) == 0 ? work_deal(p.interleave, p.G, nqb, total >> 3, p.causal != 0 || p.mask != nullptr) : 0;
    constexpr bool DENSE = MASK == 1 || MASK == 3;
    if constexpr (MASK == 0 && NW == 4) {
        if (p.num_splits > 1) {          // split launch: partial results, then the split-KV kernels' combine pass
            hipLaunchKernelGGL((sdpa_prefill_mfma_kernel<T, D, 0, 4, true>), dim3((unsigned)total, (unsigned)p.num_splits), dim3(256), 0, stream, p);
            hipError_t e = hipGetLastError();
            return e != hipSuccess ? e : launch_sdpa_combine(p, std::is_same<T, f16_t>::value ? 1 : 2, stream);
        }
    }
    if constexpr (MASK == 0 && D == 128) {
        if (p.D <= 96 && p.Dv <= 96) {   // the last quarter of the layout is padding: the instance that leaves it out of the products
            hipLaunchKernelGGL((sdpa_prefill_mfma_kernel<T, D, 0, NW, false, 6, 3>), dim3((unsigned)total), dim3(64 * NW), 0, stream, p);
            return hipGetLastError();
        }
    }
    (void)DENSE;
    hipLaunchKernelGGL((sdpa_prefill_mfma_kernel<T, D, MASK, NW>), dim3((unsigned)total), dim3(64 * NW), 0, stream, p);
    return hipGetLastError();
}

// 256-row workgroups where there is work enough for them (measured: level with 128-row workgroups at six 256-row blocks per
// compute unit and 2048 keys, 2 - 3.5 % ahead from 4096 keys on, far behind when the launch does not fill the device) -
// head dimension 128 without a dense mask (with one the 256-row form is 6 % behind: the wavefronts of a workgroup see
// different stretches of the mask and wait for each other at every tile); 128-row workgroups otherwise.
// With a dense mask (MASK = 1): first the launch for the blocks whose rows all have a limit (MASK = 2, in the form the rule
// picks), then the 128-row launch that reads the mask, for the others.
template <typename T, int D, int MASK>
static hipError_t launch_prefill_t(const SdpaParams& p0, hipStream_t stream)
{
    SdpaParams p = p0;
    if constexpr (MASK == 1) {
        if (p.mask_lims != nullptr) {
            hipError_t e = launch_prefill_t<T, D, 2>(p, stream);
            if (e != hipSuccess) return e;
            const char* forced = getenv("INCIN_ROCM_PREFILL_BLOCK_ROWS");      // (the same rule as below: the block the first launch took)
            const int rows = forced ? atoi(forced) : 0;
            const int64_t blocks256 = (int64_t)((p.Sq + 255) / 256) * p.Hq * p.B;
            p.lims_rows = D == 128 && (rows == 256 || (rows != 128 && p.Skv >= 4096 && blocks256 >= 6 * (int64_t)device_cus())) ? 256 : 128;
        }
        // the mask's values through LDS where its layout allows the copies; at D = 128 in workgroups of 256 rows (the buffers
        // of two workgroups of 128 would not fit a compute unit beside their K and V tiles)
        if (p.mask_chunks) return launch_prefill_nw<T, D, 3, D == 128 ? 8 : 4>(p, stream);
    }
    if constexpr (D == 128 && MASK != 1) {
        // INCIN_ROCM_PREFILL_BLOCK_ROWS = 128 or 256 overrides the rule (for tests: small shapes through the 256-row form)
        const char* forced = getenv("INCIN_ROCM_PREFILL_BLOCK_ROWS");
        const int rows = forced ? atoi(forced) : 0;
        const int64_t blocks256 = (int64_t)((p.Sq + 255) / 256) * p.Hq * p.B;
        if (p.num_splits <= 1 && (rows == 256 || (rows != 128 && p.Skv >= 4096 && blocks256 >= 6 * (int64_t)device_cus()))) {
            p.lims_rows = 256;
            return launch_prefill_nw<T, D, MASK, 8>(p, stream);
        }
    }
    if constexpr (MASK == 2) p.lims_rows = 128;
    return launch_prefill_nw<T, D, MASK, 4>(p, stream);
}

// Host has validated: dtype f16/bf16, D and Dv <= 128 in whole 16-byte vectors (p.Dp = the instance: 64 or 128), scale > 0, rows 16-byte aligned with unit last-dim stride, row strides below 2^24
// elements (tile offsets fit the 32-bit buffer offset).
hipError_t launch_sdpa_prefill_mfma(const SdpaParams& p, int dtype, hipStream_t stream)
{
    if (p.mask) {
        if (dtype == 1) return p.Dp == 128 ? launch_prefill_t<f16_t, 128, 1>(p, stream) : launch_prefill_t<f16_t, 64, 1>(p, stream);
        return p.Dp == 128 ? launch_prefill_t<bf16_t, 128, 1>(p, stream) : launch_prefill_t<bf16_t, 64, 1>(p, stream);
    }
    if (dtype == 1) return p.Dp == 128 ? launch_prefill_t<f16_t, 128, 0>(p, stream) : launch_prefill_t<f16_t, 64, 0>(p, stream);
    return p.Dp == 128 ? launch_prefill_t<bf16_t, 128, 0>(p, stream) : launch_prefill_t<bf16_t, 64, 0>(p, stream);
}

}  // namespace incin_rocm
