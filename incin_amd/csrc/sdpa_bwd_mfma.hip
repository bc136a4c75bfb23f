// bf16 / f16 attention backward on the gfx950 matrix cores, head dimension 64 or 128 (described for 128): dQ, dK, dV of
// O = softmax(Q K^T s + mask) V for an upstream gradient dO, from Q, K, V, O, dO and the forward's row
// normalisers L_i = log sum_j exp(x_ij) (the reference reaches the same gradients by walking its tape of
// composed ops: crates/incin-backends/src/cpu/ops/matmul.rs:264-281, cpu/ops/elementwise.rs:1062-1077).
//
//   P_ij = exp(x_ij - L_i)      dP_ij = dO_i . V_j      D_i = dO_i . O_i      dS_ij = P_ij (dP_ij - D_i)
//   dV_j = sum_i P_ij dO_i      dK_j = s sum_i dS_ij Q_i      dQ_i = s sum_j dS_ij K_j
//
// Three kernels, no atomics, P and dP recomputed in both big ones:
//   sdpa_bwd_delta_kernel   per query row, into the workspace: -L_i log2(e) and -D_i (f32), the values both big kernels
//                           start their S and dP accumulators from
//   sdpa_bwd_dq_kernel      the forward's shape of work: a wavefront owns 32 query rows (Q and dO rows resident in
//                           registers), K / V tiles stream through LDS; S^T = K Q'^T and dP^T = V dO^T have the
//                           lane-owns-a-query accumulator layout of the forward, which is again the B-operand layout
//                           of the next product, dQ^T += K^T dS^T (K^T through the transposing LDS read)
//   sdpa_bwd_dkv_kernel     the same with the roles swapped: a pair of wavefronts owns 32 keys (K and V rows resident),
//                           Q / dO tiles of the group's query heads stream through LDS; S = Q K'^T and dP = dO V^T have a
//                           lane-owns-a-key layout, the B-operand layout of dV^T += dO^T P and dK^T += Q^T dS
#include <type_traits>

#include "sdpa_bwd.h"
#include "sdpa_mfma_common.h"
#include "side_stream.h"

namespace incin_rocm {

// ---- D_i = dO_i . O_i ---------------------------------------------------------------------------------------------
// Sixteen lanes per row (16 bytes of O and of dO each), four rows per wavefront.
template <typename T>
__global__ __launch_bounds__(256) void sdpa_bwd_delta_kernel(SdpaBwdParams p)
{
    typedef typename Mma<T>::vec8 vec8;
    const int lane = threadIdx.x & 63, sub = lane & 15;
    const int64_t row = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 4 + (lane >> 4);     // (b * Hq + hq) * Sq + i
    const int64_t rows = (int64_t)p.f.B * p.f.Hq * p.f.Sq;
    float acc = 0.0f;
    if (row < rows) {
        const int i = (int)(row % p.f.Sq);
        const int64_t bh = row / p.f.Sq;
        const int hq = (int)(bh % p.f.Hq), b = (int)(bh / p.f.Hq);
        const T* o = (const T*)p.f.o + b * p.f.o_sb + hq * p.f.o_sh + (int64_t)i * p.f.o_ss;
        const T* g = (const T*)p.d_o + b * p.do_sb + hq * p.do_sh + (int64_t)i * p.do_ss;
        for (int d = sub * 8; d < p.f.Dv; d += 128) {
            const vec8 x = *(const vec8*)(o + d), y = *(const vec8*)(g + d);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc = fmaf((float)x[e], (float)y[e], acc);
        }
    }
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (row < rows && sub == 0) {
        // A row without a visible key (L_i = -inf, O and so D_i NaN) gets -inf and 0: its P is then 0 everywhere.
        const float l = p.f.lse[row];
        p.neg_delta[row] = l == -INFINITY ? 0.0f : -acc;
        p.neg_l2[row] = l == -INFINITY ? -INFINITY : -l * 1.4426950408889634f;
    }
}

// What both big kernels share: 64-row tiles of two tensors streamed through LDS in the layout of the forward's K tiles
// (rows of 256 bytes, 16-byte chunks XOR-swizzled by fk), read either by rows (16 bytes of one row per lane: an A
// operand whose M index is the row) or transposed (the gfx950 transposing read: an A operand whose M index is the
// column block).  fk serves both reads without bank conflicts: 16 consecutive rows put one logical chunk into 16
// different slots, and the 4 rows x 64 bytes a half-wavefront transposes land in 4 different 64-byte column groups.
template <typename T, int D, int NW, int NDBU>      // NW wavefronts share a tile copy; a wavefront transposes NDBU column blocks
struct BwdTiles {
    typedef typename Mma<T>::vec8 vec8;
    typedef PfLayout<D> L;
    static constexpr int NSTEP = D / 16, LPW = L::TILE_BYTES / 1024 / NW;

    int row_addr[NSTEP];           // [k-step]: byte offset of this lane's 16 bytes of row ql, chunk 2*s + g
    int tr_addr[NDBU][2];          // [column block - db0][half]: byte offset of the transposing read
    int voff[2][LPW];              // [tensor][load]: global byte offset of this lane's 16 bytes of a tile

    int width[2];                  // [tensor]: elements of data per row (a row's chunks beyond arrive as zeros: dma_chunk_offset)

    __device__ __forceinline__ void init(int wave, int lane, int64_t stride0, int64_t stride1, int width0, int width1, int db0)
    {
        width[0] = width0;
        width[1] = width1;
        const int ql = lane & 31, g = lane >> 5, n = lane & 15, dh = (lane >> 4) & 1;
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
            row_addr[s] = ql * L::ROWB + (((2 * s + g) ^ L::fk(ql)) << 4);
        }
#pragma unroll
        for (int db = 0; db < NDBU; ++db)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int r = 8 * h + 4 * g + (n >> 2);
                const int chunk = 4 * (db0 + db) + 2 * dh + ((n & 3) >> 1);
                tr_addr[db][h] = r * L::ROWB + ((chunk ^ L::fk(r)) << 4) + (n & 1) * 8;
            }
#pragma unroll
        for (int c = 0; c < LPW; ++c) {
            const int pos = (wave * LPW + c) * 64 + lane;
            const int row = pos / L::CPR, slot = pos % L::CPR;
            voff[0][c] = dma_chunk_offset(row, (int)stride0 * 2, slot ^ L::fk(row), width0 * 2);
            voff[1][c] = dma_chunk_offset(row, (int)stride1 * 2, slot ^ L::fk(row), width1 * 2);
        }
    }
    // start the copy of rows [row0, row0 + 64) of tensor `which` (base pointer of the head, `rows` rows of `stride`
    // elements) into `dst`; rows at and beyond `rows` arrive as zeros
    __device__ __forceinline__ void issue(int which, const T* base, int64_t stride, int rows, int row0, unsigned dst, int wave) const
    {
        int64_t rem = (int64_t)(rows - row0 - 1) * stride * 2 + width[which] * 2;
        if (rem > 0x7fffffffLL) rem = 0x7fffffffLL;
        if (rem < 0) rem = 0;
        const uint4v r = dma_descriptor((const char*)base + (int64_t)row0 * stride * 2, (int)rem);
#pragma unroll
        for (int c = 0; c < LPW; ++c) dma_copy16(r, dst + (wave * LPW + c) * 1024, voff[which][c]);
    }
    // A operand by rows: rows 32*blk + ql of the tile, k-step s
    __device__ __forceinline__ vec8 rows_op(const char* tile, int blk, int s) const
    {
        return *(const vec8*)(tile + row_addr[s] + blk * 32 * L::ROWB);
    }
    // A operand transposed: column block db0 + db (32 columns), rows 16*ks .. 16*ks + 15 of the tile in the order the
    // accumulator registers of a 16-row half hold them
    __device__ __forceinline__ vec8 tr_op(const char* tile, int db, int ks) const
    {
        short8v av;
        av.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4v __attribute__((address_space(3)))*)(tile + tr_addr[db][0] + ks * 16 * L::ROWB));
        av.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4v __attribute__((address_space(3)))*)(tile + tr_addr[db][1] + ks * 16 * L::ROWB));
        return __builtin_bit_cast(vec8, av);
    }
};

// ---- dQ ----------------------------------------------------------------------------------------------------------------
// DENSE: a dense additive mask - its values (times log2 e) are added to the scores before the exponential, fetched while
// the matrix instructions of the scores run; what the mask hides (-inf) ends as P = 0 like the causal edge.
// MASK: 0 none, 1 (DENSE) as described, 2 (STAGED) DENSE with the values through LDS where the mask's rows can be copied 16 bytes
// at a time: a wavefront owns 4 KiB behind the tiles - 32 rows x 32 keys for each half of a tile, rows of 64 bytes, their four
// 16-byte chunks XOR-swizzled by row - reads a half's values from there (four 8-byte reads per lane) and, once they are
// on the scores, copies the same half of the next tile into the place they left: the copy has most of a tile's time to
// land and no load sits inside the tile.  (The buffers of two workgroups and their tiles fill a compute unit's LDS to the
// byte: the two words of the tile-range search live in the buffers before the first copy.)
// Wavefronts per SIMD: two; three for D = 64 without a mask tensor, which fits 168 registers without a spill (48 KiB of LDS
// per workgroup: three workgroups per compute unit) - the masked instances would spill 11 - 42 registers there.
template <typename T, int D, int MASK = 0>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu((D == 64 && MASK == 0) ? 3 : 2, (D == 64 && MASK == 0) ? 3 : 2)))
void sdpa_bwd_dq_kernel(SdpaBwdParams bp)
{
    [[maybe_unused]] constexpr bool DENSE = MASK != 0, STAGED = MASK == 2;
#if defined(__HIP_DEVICE_COMPILE__)
    typedef typename Mma<T>::vec8 vec8;
    typedef PfLayout<D> L;
    constexpr int NSTEP = D / 16, NDB = D / 32;
    const SdpaParams& p = bp.f;
    __shared__ __attribute__((aligned(1024))) char smem[4 * L::TILE_BYTES + (STAGED ? 4 * 4096 : 0)];      // K buffers 0, 1, V buffers 0, 1 (, mask values)

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ql = lane & 31, g = lane >> 5;
    const int Sq = p.Sq, Skv = p.Skv;
    const int nqb = (Sq + PF_BM - 1) / PF_BM;
    // the forward's work order: an eighth of the list per XCD, query blocks longest-first, heads interleaved
    const int total = gridDim.x;
    const WorkItem wi = (total & 7) == 0 ? work_item_of_share(blockIdx.x & 7, blockIdx.x >> 3, total >> 3, p.interleave, p.G, nqb, p.deal_groups)
                                         : work_item(blockIdx.x, p.interleave, p.G, nqb);
    const int gq = wi.gq, qb = wi.qblk, bhkv = wi.bhkv;
    const int hkv = bhkv % p.Hkv, b = bhkv / p.Hkv;
    const int hq = hkv * p.G + gq;
    const int q0 = qb * PF_BM;

    const T* qp = (const T*)p.q + (int64_t)b * p.q_sb + (int64_t)hq * p.q_sh;
    const T* kp = (const T*)p.k + (int64_t)b * p.k_sb + (int64_t)hkv * p.k_sh;
    const T* vp = (const T*)p.v + (int64_t)b * p.v_sb + (int64_t)hkv * p.v_sh;
    const T* gp = (const T*)bp.d_o + (int64_t)b * bp.do_sb + (int64_t)hq * bp.do_sh;
    T* dqp = (T*)bp.d_q + (int64_t)b * bp.dq_sb + (int64_t)hq * bp.dq_sh;

    int kv_len = Skv;
    if (p.kv_lens) kv_len = clampi(p.kv_lens[b], 0, Skv);
    // query rows at and beyond rows_b are padding (q_lens): what the forward left in their O and lse, and what their dO
    // holds, is never used - their dQ is written as zero and they add nothing to dK and dV.  A lane's row stays in its
    // own column of every product here, so a padding row inside a wavefront that has real ones computes in isolation.
    const int rows_b = p.q_lens ? clampi(p.q_lens[b], 0, Sq) : Sq;
    const int coff = Skv - Sq;
    const int my_i = q0 + wave * 32 + ql;
    int j_end = kv_len, lim_lane = kv_len, lim_wave_max = kv_len;
    if (p.causal) {
        j_end = clampi(min(q0 + PF_BM - 1, rows_b - 1) + coff + 1, 0, kv_len);
        lim_lane = clampi(my_i + coff + 1, 0, kv_len);
        lim_wave_max = clampi(min(q0 + wave * 32 + 31, rows_b - 1) + coff + 1, 0, kv_len);
    }
    if (q0 >= rows_b) j_end = 0;
    if (q0 + wave * 32 >= rows_b) lim_wave_max = 0;
    int n_tiles = (j_end + PF_BN - 1) / PF_BN, t_first = 0;
    const int n_act = lim_wave_max > 0 ? (lim_wave_max + PF_BN - 1) / PF_BN : 0;
    // DENSE: the block flags of this wavefront's 32 rows, one per 32 keys (1 all zero, 2 all -inf: no values to fetch), and
    // the tiles between the first and the last key block that some row of the workgroup sees (a causal mask or a window
    // given as a tensor hides the rest of the row of tiles: those are not even copied)
    [[maybe_unused]] const uint8_t* mflags = nullptr;
    [[maybe_unused]] const int nkb32 = (Skv + 31) >> 5;
    if (DENSE && p.mask_flags) {
        int* s_seen;
        if constexpr (STAGED) s_seen = (int*)(smem + 4 * L::TILE_BYTES);
        else {
            __shared__ int s_seen_words[2];
            s_seen = s_seen_words;
        }
        const int nrb32 = (Sq + 31) >> 5;
        const uint8_t* fl = mask_flags_of(p, b, hq);
        mflags = fl + (int64_t)min((q0 >> 5) + wave, nrb32 - 1) * nkb32;
        if (tid == 0) { s_seen[0] = 0x7fffffff; s_seen[1] = -1; }
        __syncthreads();
        int lo = 0x7fffffff, hi = -1;
        for (int c = tid; c < min(2 * n_tiles, nkb32); c += 256) {
            bool seen = false;
#pragma unroll
            for (int w = 0; w < 4; ++w) seen = seen || fl[(int64_t)min((q0 >> 5) + w, nrb32 - 1) * nkb32 + c] != 2;
            if (seen) { lo = min(lo, c); hi = max(hi, c); }
        }
        if (hi >= 0) { atomicMin(&s_seen[0], lo); atomicMax(&s_seen[1], hi); }
        __syncthreads();
        t_first = s_seen[1] < 0 ? 0 : __builtin_amdgcn_readfirstlane(s_seen[0]) >> 1;
        n_tiles = s_seen[1] < 0 ? 0 : min(n_tiles, (__builtin_amdgcn_readfirstlane(s_seen[1]) >> 1) + 1);
    }

    BwdTiles<T, D, 4, NDB> tl;
    tl.init(wave, lane, p.k_ss, p.v_ss, p.D, p.Dv, 0);

    // this lane's query: Q row (scaled into log2 units, as the forward does) and dO row, the row's normaliser and D_i.  The
    // rows are fetched 16 bytes per lane, eight lanes to a 128-byte run of a row, and reach the operand layout through this
    // wavefront's 4 KiB of the V buffers (fetch_q_rows / stage_q_rows), which nothing is copied into before the barrier below.
    vec8 qreg[NSTEP], greg[NSTEP];
    const int qi = min(my_i, Sq - 1);
    const unsigned lds0 = lds_address(smem);
    if (t_first < n_tiles) tl.issue(0, kp, p.k_ss, Skv, t_first * PF_BN, lds0 + (t_first & 1) * L::TILE_BYTES, wave);
    {
        static_assert(2 * L::TILE_BYTES >= 4 * 4096, "the V buffers hold a 4 KiB staging area per wavefront");
        char* stage = smem + 2 * L::TILE_BYTES + wave * 4096;
        uint4v qraw[NSTEP / 4][4], graw[NSTEP / 4][4];
        fetch_q_rows(qraw, qp, q0 + wave * 32, Sq, p.q_ss, p.D, lane);
        fetch_q_rows(graw, gp, q0 + wave * 32, Sq, bp.do_ss, p.Dv, lane);
        stage_q_rows(qreg, qraw, stage, lane);
        stage_q_rows(greg, graw, stage, lane);
        const float c2 = p.scale * 1.4426950408889634f;
#pragma unroll
        for (int s = 0; s < NSTEP; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) qreg[s][e] = (T)((float)qreg[s][e] * c2);
    }
    __syncthreads();      // every wavefront has its rows out of the V buffers
    if (t_first < n_tiles) tl.issue(1, vp, p.v_ss, Skv, t_first * PF_BN, lds0 + (2 + (t_first & 1)) * L::TILE_BYTES, wave);
    const int64_t stat = ((int64_t)b * p.Hq + hq) * Sq + qi;
    [[maybe_unused]] const T* mrow = nullptr;      // DENSE: this lane's row of the mask
    if (DENSE) mrow = (const T*)p.mask + (int64_t)b * p.m_sb + (int64_t)hq * p.m_sh + (int64_t)qi * p.m_si;
    const float l2 = -bp.neg_l2[stat];
    const float dlt = -bp.neg_delta[stat];

    floatx16 dq_acc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) dq_acc[db][r] = 0.0f;
    // The S and dP accumulators start from -L_i log2(e) and -D_i of the lane's query (what the mask hides: from -inf, which
    // ends as P = 0 and dS = 0), so P = exp2(S) and dS = P * dP need neither a subtraction nor a select.
    floatx16 seed_s, seed_d;
#pragma unroll
    for (int r = 0; r < 16; ++r) { seed_s[r] = -l2; seed_d[r] = -dlt; }
    // first key some lane of this wavefront does not see: tiles that end at or before it need no mask
    int lim_wave_min = kv_len;
    if (p.causal) lim_wave_min = clampi(q0 + wave * 32 + coff + 1, 0, kv_len);

    // DENSE: the flags of a tile are asked for ahead of it (two tiles ahead for STAGED, which decides a tile ahead what to copy),
    // after the copies of a tile are issued, and taken behind the tile barrier, before the next copies are issued: a load that
    // is issued and consumed inside one tile makes the compiler wait for everything in flight - the next tile's copies,
    // which it does not know of, included.  Without STAGED the values of a block that has any are such loads (there are no
    // registers to hold them a tile ahead): a tile with values pays a memory latency that the second workgroup of the
    // compute unit has to cover.
    typedef T vec4 __attribute__((ext_vector_type(4)));
    [[maybe_unused]] int fv[2] = {0, 0};
    [[maybe_unused]] int f_cur[2] = {0, 0}, f_nxt[2] = {0, 0};      // STAGED: the flags of tiles t and t + 1 (fv: of t + 2, as loaded)
    [[maybe_unused]] auto tile_flags = [&](int t) __attribute__((always_inline)) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) fv[kb] = 2 * t + kb < nkb32 ? (int)mflags[2 * t + kb] : 2;
    };
    // STAGED: copy c of a half's two brings rows 16 c + lane / 4, and into position lane % 4 of the row's four chunks the chunk
    // (lane % 4) ^ (row / 4 % 4) (= (lane / 16) % 4 for both copies); the rows' 16 c, the half and the tile go into the scalar
    // offset.  The descriptor starts at the wavefront's first row and ends with the head's last row (rows past Sq deliver zeros).
    [[maybe_unused]] const unsigned m_zone = lds_address(smem) + 4 * L::TILE_BYTES + wave * 4096;
    [[maybe_unused]] const int m_cp = (int)((int64_t)(lane >> 2) * p.m_si * 2) + (((lane & 3) ^ ((lane >> 4) & 3)) << 4);
    [[maybe_unused]] const int m_rd = ql * 64 + g * 8 + (((ql >> 2) & 3) << 4);      // this lane's read position in a half, before the XOR with the chunk
    [[maybe_unused]] uint4v m_desc = {0u, 0u, 0u, 0u};
    if (STAGED) {
        const int row0 = q0 + wave * 32;
        const int64_t left = row0 < Sq ? ((int64_t)(Sq - 1 - row0) * p.m_si + Skv) * 2 : 0;
        m_desc = dma_descriptor((const T*)p.mask + (int64_t)b * p.m_sb + (int64_t)hq * p.m_sh + (int64_t)row0 * p.m_si,
                                (int)(left > 0x7fffffffLL ? 0x7fffffffLL : left));
    }
    [[maybe_unused]] auto half_copy = [&](int t, int kb) __attribute__((always_inline)) {
#pragma unroll
        for (int c = 0; c < 2; ++c) dma_copy16_at(m_desc, m_zone + kb * 2048 + c * 1024, m_cp, (t * PF_BN + kb * 32) * 2 + c * 16 * (int)p.m_si * 2);
    };
    if (DENSE && mflags && t_first < n_tiles) tile_flags(t_first);
    if (STAGED && t_first < n_tiles) {
        // (the prologue's barrier is behind: the words of the tile-range search in the first buffer are done with)
        if (mflags) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) f_cur[kb] = __builtin_amdgcn_readfirstlane(fv[kb]);
            if (t_first + 1 < n_tiles) tile_flags(t_first + 1);
        }
        if (t_first < n_act) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
                if (f_cur[kb] == 0) half_copy(t_first, kb);
        }
    }
    for (int t = t_first; t < n_tiles; ++t) {
        // K(t), V(t) have landed for everyone and everyone is done with tile t-1: the other pair of buffers is free
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        [[maybe_unused]] int flags_t[2] = {0, 0};
        if (DENSE && mflags) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                asm volatile("" : "+v"(fv[kb]));
                if (STAGED) {
                    flags_t[kb] = f_cur[kb];
                    f_nxt[kb] = t + 1 < n_tiles ? __builtin_amdgcn_readfirstlane(fv[kb]) : 2;
                } else
                    flags_t[kb] = __builtin_amdgcn_readfirstlane(fv[kb]);
            }
        }
        if (t + 1 < n_tiles) {
            tl.issue(0, kp, p.k_ss, Skv, (t + 1) * PF_BN, lds0 + ((t + 1) & 1) * L::TILE_BYTES, wave);
            tl.issue(1, vp, p.v_ss, Skv, (t + 1) * PF_BN, lds0 + (2 + ((t + 1) & 1)) * L::TILE_BYTES, wave);
            if (DENSE && mflags && !STAGED) tile_flags(t + 1);
        }
        if (STAGED && mflags) {
            if (t + 2 < n_tiles) tile_flags(t + 2);
            f_cur[0] = f_nxt[0];
            f_cur[1] = f_nxt[1];
        }
        if (t >= n_act) continue;
        const char* kt = smem + (t & 1) * L::TILE_BYTES;
        const char* vt = smem + (2 + (t & 1)) * L::TILE_BYTES;
        const int j0 = t * PF_BN;
        const bool edge = j0 + PF_BN > lim_wave_min;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            floatx16 s_acc = seed_s, dp_acc = seed_d;
            if (edge) {
                // register r is key j0 + 32*kb + 8*(r/4) + 4*g + (r%4)
                const int rel = lim_lane - (j0 + 32 * kb + 4 * g);
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (8 * (r / 4) + (r % 4) >= rel) s_acc[r] = -INFINITY;
            }
            [[maybe_unused]] vec4 mv[4];
            [[maybe_unused]] int flag = 0;
            if (DENSE && mflags) {
                flag = flags_t[kb];
                if (flag == 2) {      // the mask hides the block from all 32 rows: S starts from -inf, as at the causal edge (the
                                      // products run all the same: branches around them cost every tile more than these blocks save)
                    asm volatile("" ::: "memory");
#pragma unroll
                    for (int r = 0; r < 16; ++r) s_acc[r] = -INFINITY;
                }
            }
            if (DENSE && flag == 0) {      // the mask's values of this lane's 16 keys, asked for ahead of the products
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const int j = j0 + 32 * kb + 8 * r4 + 4 * g;
                    if (STAGED) mv[r4] = *(const vec4*)(smem + 4 * L::TILE_BYTES + wave * 4096 + kb * 2048 + (m_rd ^ (r4 << 4)));
                    else if (p.mask_vec && j + 3 < Skv) mv[r4] = *(const vec4*)(mrow + j);
                    else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) mv[r4][e] = mrow[(int64_t)min(j + e, Skv - 1) * p.m_sj];
                    }
                }
            }
#pragma unroll
            for (int s = 0; s < NSTEP; ++s) {
                s_acc = Mma<T>::run(tl.rows_op(kt, kb, s), qreg[s], s_acc);
                dp_acc = Mma<T>::run(tl.rows_op(vt, kb, s), greg[s], dp_acc);
            }
            if (DENSE && flag == 0) {
#pragma unroll
                for (int r = 0; r < 16; ++r) s_acc[r] = __builtin_fmaf((float)mv[r / 4][r % 4], 1.4426950408889634f, s_acc[r]);
            }
            if (STAGED) {      // (this half's values are on the scores: its place is free for the same half of the next tile)
                const int fn = mflags ? f_cur[kb] : 0;      // (f_cur holds the next tile's flags by now)
                if (t + 1 < n_tiles && t + 1 < n_act && fn == 0) {
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    half_copy(t + 1, kb);
                }
            }
            vec8 ds[2];
#pragma unroll
            for (int r = 0; r < 16; ++r) ds[r / 8][r % 8] = (T)(__builtin_amdgcn_exp2f(s_acc[r]) * dp_acc[r]);
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int db = 0; db < NDB; ++db) dq_acc[db] = Mma<T>::run(tl.tr_op(kt, db, 2 * kb + h), ds[h], dq_acc[db]);
        }
    }

    // dQ rows out (store_o_rows): padding rows inside Sq as zeros; staged through 4 KiB of the buffers the last tile did not
    // use (every wavefront is past that tile's barrier, i.e. done with the tile before it) - at D = 64 a buffer holds two
    // wavefronts' areas, so two wavefronts take the K buffer and two the V buffer
    if (my_i >= rows_b) {
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) dq_acc[db][r] = 0.0f;
    }
    {
        constexpr int PER_BUF = L::TILE_BYTES / 4096;      // staging areas per buffer: 4 (D = 128) or 2
        char* stage = smem + ((wave / PER_BUF) * 2 + (max(n_tiles, t_first) & 1)) * L::TILE_BYTES + (wave % PER_BUF) * 4096;
        store_o_rows(dq_acc, p.scale, stage, dqp, q0 + wave * 32, Sq, bp.dq_ss, p.D, lane);
    }
#endif
}

// ---- dK, dV ---------------------------------------------------------------------------------------------------------------
constexpr int BWD_KEYS = 128;      // keys per workgroup of the dK/dV kernel
constexpr int BWD_RING = 4;        // matrix operands in flight from LDS (reads run this many matrix instructions ahead)

// A wavefront that has a SIMD to itself pays for every instruction it issues on top of its matrix instructions (nothing
// of its own overlaps them), and 32 keys' dK and dV (128 accumulators) with the K and V rows (64 registers) and a tile's
// S and dP leave no room for a second one.  So two wavefronts share each block of 32 keys, eight per workgroup, two
// per SIMD, and split a 64-query tile both ways:
//   first   S and dP of ONE 32-row query block (16 matrix instructions), P and dS from them, written to LDS;
//   then    dV and dK of the 32 keys for ONE half of the head dimension, over both query blocks (16 matrix
//           instructions; P and dS of both blocks come back from LDS, the partner's and the wavefront's own).
// Each holds 64 accumulators and the matrix work is not duplicated.  The two halves are pipelined over tiles: a step
// computes S, dP of tile t, then dV, dK of tile t - 1 with the exponentials and products that make P, dS of tile t
// issued between those matrix instructions (the workgroup's barriers keep the two wavefronts of a SIMD in the same
// phase, so what overlaps a wavefront's matrix instructions has to come from its own stream), and writes P, dS of tile
// t after a barrier.  Tiles t - 1 and t stay resident while tile t + 1 is copied: three stages.  The S and dP
// accumulators do not start from zero but from -L_i log2(e) and -D_i (staged per tile next to the Q and dO rows), so
// P = exp2(S) and dS = P * dP need no subtraction.
// DENSE: a dense additive mask, with one flag per block of 32 rows x 32 keys (mask_classify_kernel ran before).  Tiles before
// the first and after the last block that shows this workgroup any key are left out; inside that range a block of zeros or
// of -inf needs no values.  Otherwise: a lane holds one key and 16 query rows of a block, so its mask values are 16 loads down a
// column of the mask, asked for at the start of a step and added (times log2 e) to the scores where P is taken.
// MASK: 0 none, 1 (DENSE) as described, 2 (STAGED) DENSE with the values through LDS where the mask's rows can be copied 16 bytes
// at a time: every wavefront copies the 32 rows x 32 keys of its own block of the next tile (two copies, rows of 64 bytes) into
// 2 KiB of its own and takes its column of them with four transposing reads - 8 bytes per lane, four rows of four keys,
// handed round among 16 lanes so that each ends with four rows of its own key - instead of 16 two-byte loads.
template <typename T, int D, int MASK = 0>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void sdpa_bwd_dkv_kernel(SdpaBwdParams bp)
{
    [[maybe_unused]] constexpr bool DENSE = MASK != 0, STAGED = MASK == 2;
#if defined(__HIP_DEVICE_COMPILE__)
    typedef typename Mma<T>::vec8 vec8;
    typedef PfLayout<D> L;
    typedef float float4v __attribute__((ext_vector_type(4)));
    constexpr int NSTEP = D / 16, R = BWD_RING;
    constexpr int NCB = D / 64;                         // 32-wide column blocks of dK / dV per wavefront (its half of the head dimension)
    constexpr int NA = 2 * NSTEP;                       // matrix instructions of the first half of a step (S and dP)
    constexpr int NB2 = 8 * NCB;                        // of the second half: 4 groups of 16 query rows x NCB blocks x (dV, dK)
    constexpr int STAGE = 2 * L::TILE_BYTES + 1024;     // Q rows, dO rows, 64 x -L_i log2(e), 64 x -D_i (and padding)
    constexpr int XCHG = 4 * 2 * 4 * 1024;              // [key block][query block][P lo, P hi, dS lo, dS hi]: 64 lanes x 16 bytes
    const SdpaParams& p = bp.f;
    constexpr int NS = 3;                               // stages: tiles t - 1 and t in use, tile t + 1 arriving
    constexpr int MZONE = STAGED ? 8 * 2048 : 0;        // STAGED: 32 rows x 64 bytes of mask values per wavefront
    __shared__ __attribute__((aligned(1024))) char smem[NS * STAGE + XCHG + MZONE];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kb = wave & 3;           // block of 32 keys
    const int role = wave >> 2;        // query block of the first half, half of the head dimension of the second
    const int ql = lane & 31, g = lane >> 5;
    const int Sq = p.Sq, Skv = p.Skv;
    const int nkb = (Skv + BWD_KEYS - 1) / BWD_KEYS;
    // Workgroups reach the 8 XCDs round-robin by id.  All key blocks of a (batch, KV head) pair read the same Q and dO
    // rows, so a pair is given to one XCD (pair h to XCD h % 8) and its key blocks run there side by side, the
    // block with the most visible queries (the first, under a causal mask) first.
    int kblk, bhkv;
    {
        const int pairs = p.B * p.Hkv;
        if ((pairs & 7) == 0) {
            const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
            kblk = slot % nkb;
            bhkv = (slot / nkb) * 8 + xcd;
        } else {
            kblk = blockIdx.x % nkb;
            bhkv = blockIdx.x / nkb;
        }
    }
    const int hkv = bhkv % p.Hkv, b = bhkv / p.Hkv;
    const int j0 = kblk * BWD_KEYS;
    const int my_j = j0 + kb * 32 + ql;                // this lane's key

    const T* kp = (const T*)p.k + (int64_t)b * p.k_sb + (int64_t)hkv * p.k_sh;
    const T* vp = (const T*)p.v + (int64_t)b * p.v_sb + (int64_t)hkv * p.v_sh;
    T* dkp = (T*)bp.d_k + (int64_t)b * bp.dk_sb + (int64_t)hkv * bp.dk_sh;
    T* dvp = (T*)bp.d_v + (int64_t)b * bp.dv_sb + (int64_t)hkv * bp.dv_sh;

    int kv_len = Skv;
    if (p.kv_lens) kv_len = clampi(p.kv_lens[b], 0, Skv);
    const int coff = Skv - Sq;
    // query rows that see any key of this workgroup: i >= j - coff for its first key (causal)
    const int i_begin_wg = p.causal ? clampi(j0 - coff, 0, Sq) : 0;
    // first query row that sees every key of this wavefront: tiles from there on need no mask
    const int i_all_wave = p.causal ? max(j0 + kb * 32 + 31 - coff, 0) : 0;
    int t_begin = i_begin_wg / PF_BN;
    // query rows at and beyond rows_b are padding (q_lens): the tiles end there, and the rows between there and the end of
    // the last tile arrive as zeros like rows past Sq (Q, dO and the per-row values), which leaves dS and P^T dO at zero
    const int rows_b = p.q_lens ? clampi(p.q_lens[b], 0, Sq) : Sq;
    int n_qt = (rows_b + PF_BN - 1) / PF_BN;
    if (DENSE && p.mask_flags) {
        // The tiles between the first and the last block of 32 query rows, over the group's heads, from which the mask does not
        // hide all of this workgroup's keys: a causal mask or a window given as a tensor leaves the others out altogether.
        __shared__ int s_seen[2];
        const int nkb = (Skv + 31) >> 5, nrb = (Sq + 31) >> 5, c0 = kblk * 4;
        if (tid == 0) { s_seen[0] = 0x7fffffff; s_seen[1] = -1; }
        __syncthreads();
        int lo = 0x7fffffff, hi = -1;
        const int r_lo = 2 * t_begin, r_n = min(2 * n_qt, nrb) - r_lo;
        for (int x = tid; x < r_n * p.G; x += 512) {
            const int rb = r_lo + x % r_n;
            const uint8_t* fl = mask_flags_of(p, b, hkv * p.G + x / r_n) + (int64_t)rb * nkb;
            bool seen = false;
#pragma unroll
            for (int c = 0; c < 4; ++c) seen = seen || fl[min(c0 + c, nkb - 1)] != 2;
            if (seen) { lo = min(lo, rb); hi = max(hi, rb); }
        }
        if (hi >= 0) { atomicMin(&s_seen[0], lo); atomicMax(&s_seen[1], hi); }
        __syncthreads();
        if (s_seen[1] < 0) n_qt = t_begin;
        else {
            t_begin = __builtin_amdgcn_readfirstlane(s_seen[0]) >> 1;
            n_qt = (__builtin_amdgcn_readfirstlane(s_seen[1]) >> 1) + 1;
        }
    }
    const int tiles_per_head = j0 < kv_len ? max(n_qt - t_begin, 0) : 0;
    const int n_all = tiles_per_head * p.G;             // the group's query heads one after another
    // bp.parts_kv workgroups share a key block: each walks a stretch n_lo .. n_tiles - 1 of the tiles and leaves its sums in a
    // plane of the workspace (blockIdx.y says which stretch; one workgroup: the whole walk, and the gradients' rows directly)
    const int part = blockIdx.y, parts = gridDim.y;
    const int n_lo = parts > 1 ? (int)((int64_t)n_all * part / parts) : 0;
    const int n_tiles = parts > 1 ? (int)((int64_t)n_all * (part + 1) / parts) : n_all;

    BwdTiles<T, D, 8, NCB> tl;
    tl.init(wave, lane, p.q_ss, bp.do_ss, p.D, p.Dv, NCB * role);

    // this lane's key: K row (scaled into log2 units) and V row as B operands
    vec8 kreg[NSTEP], vreg[NSTEP];
    {
        const int kj = min(my_j, Skv - 1);
        const T* krow = kp + (int64_t)kj * p.k_ss + g * 8;
        const T* vrow = vp + (int64_t)kj * p.v_ss + g * 8;
        const float c2 = p.scale * 1.4426950408889634f;
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
            vec8 x, y;
#pragma unroll
            for (int e = 0; e < 8; ++e) { x[e] = (T)0.0f; y[e] = (T)0.0f; }
            if (s * 16 + g * 8 < p.D) x = *(const vec8*)(krow + s * 16);
            if (s * 16 + g * 8 < p.Dv) y = *(const vec8*)(vrow + s * 16);
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = (T)((float)x[e] * c2);
            kreg[s] = x;
            vreg[s] = y;
        }
    }
    // rows i >= lo_i see this lane's key under the causal mask
    const int lo_i = p.causal ? my_j - coff : -0x40000000;

    floatx16 dk_acc[NCB], dv_acc[NCB];     // column blocks NCB * role .. NCB * role + NCB - 1
#pragma unroll
    for (int d = 0; d < NCB; ++d)
#pragma unroll
        for (int r = 0; r < 16; ++r) { dk_acc[d][r] = 0.0f; dv_acc[d][r] = 0.0f; }

    // The copies walk the tiles with running addresses instead of index arithmetic per tile.
    const unsigned lds0 = lds_address(smem);
    const int64_t q_step = (int64_t)PF_BN * p.q_ss * 2, g_step = (int64_t)PF_BN * bp.do_ss * 2;
    const char *nx_q = nullptr, *nx_g = nullptr, *nx_s = nullptr;      // next tile to copy: Q rows, dO rows, per-row floats
    int64_t nx_qrem = 0, nx_grem = 0;                                  // bytes from there to the end of the last row
    int nx_rows = 0, nx_r = 0, nx_h = 0;                               // rows left, tile within the head, head within the group
    auto to_head = [&](int h) __attribute__((always_inline)) {
        const int hq = hkv * p.G + h, r0 = t_begin * PF_BN;
        nx_q = (const char*)p.q + ((int64_t)b * p.q_sb + (int64_t)hq * p.q_sh + (int64_t)r0 * p.q_ss) * 2;
        nx_g = (const char*)bp.d_o + ((int64_t)b * bp.do_sb + (int64_t)hq * bp.do_sh + (int64_t)r0 * bp.do_ss) * 2;
        nx_s = (const char*)((wave == 0 ? bp.neg_l2 : bp.neg_delta) + ((int64_t)b * p.Hq + hq) * Sq + r0);
        nx_rows = rows_b - r0;
        nx_qrem = (int64_t)(nx_rows - 1) * p.q_ss * 2 + p.D * 2;
        nx_grem = (int64_t)(nx_rows - 1) * bp.do_ss * 2 + p.Dv * 2;
        nx_r = 0;
        nx_h = h;
    };
    auto seek = [&](int n) __attribute__((always_inline)) {      // the copies start at tile n of the walk
        const int h = n / tiles_per_head, r = n - h * tiles_per_head;
        to_head(h);
        nx_q += r * q_step; nx_g += r * g_step; nx_s += (int64_t)r * PF_BN * 4;
        nx_qrem -= r * q_step; nx_grem -= r * g_step; nx_rows -= r * PF_BN;
        nx_r = r;
    };
    auto clamp31 = [](int64_t x) { return (x >> 31) ? 0x7fffffff : (int)x; };       // (x is never negative here)
    auto issue = [&](int stage) __attribute__((always_inline)) {
        const unsigned st = lds0 + stage * STAGE;
        const uint4v dq_ = dma_descriptor(nx_q, clamp31(nx_qrem)), dg_ = dma_descriptor(nx_g, clamp31(nx_grem));
#pragma unroll
        for (int c = 0; c < tl.LPW; ++c) dma_copy16(dq_, st + (wave * tl.LPW + c) * 1024, tl.voff[0][c]);
#pragma unroll
        for (int c = 0; c < tl.LPW; ++c) dma_copy16(dg_, st + L::TILE_BYTES + (wave * tl.LPW + c) * 1024, tl.voff[1][c]);
        if (wave < 2)           // 64 floats of one of the two per-row arrays; rows past Sq arrive as zeros
            dma_copy4(dma_descriptor(nx_s, nx_rows * 4), st + 2 * L::TILE_BYTES + wave * 256, lane * 4);
        if (++nx_r == tiles_per_head) {
            if (nx_h + 1 < p.G) to_head(nx_h + 1);
        } else {
            nx_q += q_step; nx_g += g_step; nx_s += PF_BN * 4;
            nx_qrem -= q_step; nx_grem -= g_step; nx_rows -= PF_BN;
        }
    };

    char* const xmine = smem + NS * STAGE + ((kb * 2 + role) * 4) * 1024 + lane * 16;
    const char* const xother = smem + NS * STAGE + ((kb * 2 + 1 - role) * 4) * 1024 + lane * 16;
    const int own_rows = role * 32 * L::ROWB, other_rows = (1 - role) * 32 * L::ROWB;

    // One step of the pipeline: S, dP of tile t (16 matrix instructions), then dV, dK of tile t - 1 (16 more, operands from
    // that tile's stage and from the exchange buffer) with P and dS of tile t computed on the vector ALU between them, then
    // - after a barrier, when everyone has read tile t - 1's P and dS - this wavefront's P and dS of tile t into the buffer.
    // WITH_A = false is the step after the last tile: only the second half.
    // DENSE: the mask's column of this lane's key, for the query head in hand; and the flags of this wavefront's 32 keys -
    // per block of 32 query rows: 1 says the mask is zero there, 2 that it hides the keys from all of the rows (neither needs
    // the mask's values)
    // (the values are fetched with one lane offset - the key's column and the lane's first row - plus a scalar offset per
    // register, from a descriptor that starts at the tile's first row and ends with the head's last row: rows past Sq read
    // zeros; the host has checked that 64 rows fit 32-bit offsets)
    [[maybe_unused]] const int m_lane = (int)(((int64_t)min(my_j, Skv - 1) * p.m_sj + (int64_t)(4 * g) * p.m_si) * 2);
    [[maybe_unused]] const int m_row2 = (int)(p.m_si * 2);
    [[maybe_unused]] const int nkb32 = (Skv + 31) >> 5, nrb32 = (Sq + 31) >> 5;
    [[maybe_unused]] const int my_kb32 = min(kblk * 4 + kb, nkb32 - 1);
    // The flag of a tile (this wavefront's query block of it) is asked for two tiles ahead and the values of a block that has
    // any one tile ahead, right after the copies of that tile are issued, into registers of their own that are handed over
    // behind the tile barrier: a load that is issued and consumed inside one step makes the compiler wait for everything in
    // flight - the next tile's copies, which it does not know of, included: a memory latency in every step.
    typedef T vec2 __attribute__((ext_vector_type(2)));
    // (each value arrives in a register of its own - a 16-bit load into half a register would have to wait for the load
    // of the other half - and two are packed into one at the hand-over)
    [[maybe_unused]] vec2 mval[8];
    [[maybe_unused]] unsigned mnext[16];
    [[maybe_unused]] auto tile_of = [&](int n, int* i0, int* head) __attribute__((always_inline)) {       // n-th tile of the walk
        *head = n / tiles_per_head;
        *i0 = (t_begin + n % tiles_per_head) * PF_BN;
    };
    [[maybe_unused]] auto tile_flag = [&](int n) __attribute__((always_inline)) {
        int i0, head;
        tile_of(n, &i0, &head);
        return (int)mask_flags_of(p, b, hkv * p.G + head)[(int64_t)min((i0 >> 5) + role, nrb32 - 1) * nkb32 + my_kb32];
    };
    // STAGED: copy c of a tile's two brings rows 16 c + lane / 4, 16-byte chunk lane % 4 of the 64 bytes this wavefront's 32 keys
    // take in a row (the rows' 16 c into the scalar offset); the descriptor starts at the block's first row and first key and
    // ends with the head's last row, so rows past Sq deliver zeros.  A lane's transposing read r4 takes 8 bytes of row
    // 8 r4 + 4 g + (lane % 16) / 4, keys 16 (lane / 16 % 2) + 4 (lane % 4) .. + 3, and returns rows 8 r4 + 4 g .. + 3 of key lane % 32.
    [[maybe_unused]] const unsigned m_zone = lds_address(smem) + NS * STAGE + XCHG + wave * 2048;
    [[maybe_unused]] const int m_cp = (int)((int64_t)(lane >> 2) * p.m_si * 2) + (lane & 3) * 16;
    [[maybe_unused]] const int m_tr = (4 * g + ((lane & 15) >> 2)) * 64 + ((lane >> 4) & 1) * 32 + (lane & 3) * 8;
    [[maybe_unused]] auto tile_copy = [&](int n) __attribute__((always_inline)) {
        int i0, head;
        tile_of(n, &i0, &head);
        const int row0 = i0 + 32 * role, key0 = j0 + kb * 32;
        const T* mc = (const T*)p.mask + (int64_t)b * p.m_sb + (int64_t)(hkv * p.G + head) * p.m_sh + (int64_t)row0 * p.m_si + key0;
        const int64_t left = row0 < Sq && key0 < Skv ? ((int64_t)(Sq - 1 - row0) * p.m_si + (Skv - key0)) * 2 : 0;
        const uint4v md = dma_descriptor(mc, (int)min(left, (int64_t)0x7fffffff));
#pragma unroll
        for (int c = 0; c < 2; ++c) dma_copy16_at(md, m_zone + c * 1024, m_cp, c * 16 * (int)p.m_si * 2);
    };
    [[maybe_unused]] auto tile_values = [&](int n) __attribute__((always_inline)) {      // register r is row i0 + 32 * role + 8 * (r / 4) + 4 * g + (r % 4)
        int i0, head;
        tile_of(n, &i0, &head);
        const int row0 = i0 + 32 * role;
        const T* mc = (const T*)p.mask + (int64_t)b * p.m_sb + (int64_t)(hkv * p.G + head) * p.m_sh + (int64_t)row0 * p.m_si;
        const int64_t left = row0 < Sq ? ((int64_t)(Sq - 1 - row0) * p.m_si + (int64_t)(Skv - 1) * p.m_sj + 1) * 2 : 0;
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)mc, 0, (int)min(left, (int64_t)0x7fffffff), 0x00020000);
#pragma unroll
        for (int r = 0; r < 16; ++r)
            mnext[r] = (unsigned short)__builtin_amdgcn_raw_buffer_load_b16(rs, m_lane, (8 * (r / 4) + (r % 4)) * m_row2, 0);
    };
    auto step = [&](int stage, int pstage, int i0, bool has_prev, [[maybe_unused]] int f_own, auto WITH_A_) __attribute__((always_inline)) {
        constexpr bool WITH_A = decltype(WITH_A_)::value;
        const char* qt = smem + stage * STAGE;
        const char* gt = qt + L::TILE_BYTES;
        const char* nl = gt + L::TILE_BYTES + role * 128;
        const char* pq = smem + pstage * STAGE;
        const char* pg = pq + L::TILE_BYTES;
        vec8 ring[R];
        floatx16 sa, da;
        vec8 pp[2], ds[2];
        [[maybe_unused]] bool own_hidden = false, own_zero = false;
        if (WITH_A && DENSE) {
            own_hidden = f_own == 2;
            own_zero = f_own == 1;
        }
        [[maybe_unused]] const bool own_values = WITH_A && DENSE && !own_zero && !own_hidden;
        if (WITH_A) {
            // The accumulators start from -L_i log2(e) and -D_i.  What the mask hides starts from -inf instead and ends as
            // P = 0, dS = 0 * (finite): only the causal edge needs that here, rows past Sq arrive as zeros throughout (dO = 0,
            // dP = 0), rows without any visible key carry -inf already, and keys past kv_len are zeroed at the end.
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const float4v a = *(const float4v*)(nl + (8 * r4 + 4 * g) * 4);
                const float4v d = *(const float4v*)(nl + 256 + (8 * r4 + 4 * g) * 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) { sa[4 * r4 + e] = a[e]; da[4 * r4 + e] = d[e]; }
            }
            // S (even i) and dP (odd i) of the own query block, k-step i / 2
            auto fetch_a = [&](int i) __attribute__((always_inline)) {
                ring[i % R] = *(const vec8*)((i % 2 ? gt : qt) + own_rows + tl.row_addr[i / 2]);
            };
#pragma unroll
            for (int i = 0; i < R; ++i) fetch_a(i);
            if (DENSE && own_hidden) {      // (as at the causal edge: S starts from -inf; the products run all the same - branches
                                            //  around them cost every tile more than these tiles save)
                asm volatile("" ::: "memory");
#pragma unroll
                for (int r = 0; r < 16; ++r) sa[r] = -INFINITY;
            }
            if (i0 < i_all_wave) {          // some row of the tile does not see every key of this wavefront
                asm volatile("" ::: "memory");      // (a real branch: as selects this would cost every tile 32 vector instructions)
                const int rel = lo_i - i0 - 4 * g - 32 * role;      // register r is row i0 + 32*role + 8*(r/4) + 4*g + (r%4)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (8 * (r / 4) + (r % 4) < rel) sa[r] = -INFINITY;
            }
#pragma unroll
            for (int i = 0; i < NA; ++i) {
                if (i % 2 == 0) sa = Mma<T>::run(ring[i % R], kreg[i / 2], sa);
                else da = Mma<T>::run(ring[i % R], vreg[i / 2], da);
                if (i + R < NA) fetch_a(i + R);
            }
            if (own_values) {       // (the mask's values are no longer needed past this point: the second half has no room for them)
#pragma unroll
                for (int r = 0; r < 16; ++r) sa[r] = __builtin_fmaf((float)mval[r / 2][r % 2], 1.4426950408889634f, sa[r]);
            }
        }
        // P and dS of register r of the own query block, rounded for the next products
        auto soft = [&](int r) __attribute__((always_inline)) {
            if (!WITH_A) return;
            const float pr = __builtin_amdgcn_exp2f(sa[r]);
            pp[r / 8][r % 8] = (T)pr;
            ds[r / 8][r % 8] = (T)(pr * da[r]);
        };
        if (has_prev) {
            // Matrix instruction m of the second half: group m / (2 NCB) = (own query block, rows 0-15), (own, 16-31),
            // (partner's, 0-15), (partner's, 16-31); column block (m / 2) % NCB of this wavefront's; dV from dO^T and P (even m),
            // dK from Q^T and dS (odd).
            auto fetch_b = [&](int m) __attribute__((always_inline)) {
                const int grp = m / (2 * NCB);
                ring[m % R] = tl.tr_op((m % 2 ? pq : pg) + (grp < 2 ? own_rows : other_rows), (m / 2) % NCB, grp % 2);
            };
            vec8 bp_[2], bs_[2];        // P and dS of a group, two groups in flight
            auto fetch_group = [&](int grp) __attribute__((always_inline)) {
                const char* x = (grp < 2 ? (const char*)xmine : xother) + (grp % 2) * 1024;
                bp_[grp % 2] = *(const vec8*)x;
                bs_[grp % 2] = *(const vec8*)(x + 2048);
            };
            fetch_group(0);
            fetch_group(1);
#pragma unroll
            for (int m = 0; m < R; ++m) fetch_b(m);
#pragma unroll
            for (int m = 0; m < NB2; ++m) {
                const int d = (m / 2) % NCB, grp = m / (2 * NCB);
                if (m % 2 == 0) dv_acc[d] = Mma<T>::run(ring[m % R], bp_[grp % 2], dv_acc[d]);
                else dk_acc[d] = Mma<T>::run(ring[m % R], bs_[grp % 2], dk_acc[d]);
                if (m + R < NB2) fetch_b(m + R);
                if (m % (2 * NCB) == 2 * NCB - 1 && grp + 2 < 4) fetch_group(grp + 2);
#pragma unroll
                for (int r = m * (16 / NB2); r < (m + 1) * (16 / NB2); ++r) soft(r);
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) soft(r);
        }
        if (WITH_A) {
            __syncthreads();            // everyone has read the previous tile's P and dS
            *(vec8*)(xmine) = pp[0];
            *(vec8*)(xmine + 1024) = pp[1];
            *(vec8*)(xmine + 2048) = ds[0];
            *(vec8*)(xmine + 3072) = ds[1];
        }
    };

    if (n_lo < n_tiles) {
        seek(n_lo);
        issue(0);
    }
    int i0 = (t_begin + (n_lo < n_tiles ? n_lo % tiles_per_head : 0)) * PF_BN, stage = 0, pstage = 0;
    // DENSE: the flags of tiles t and t + 1 (known), of tile t + 2 (asked for); without flags every block counts as one with values
    [[maybe_unused]] int f_cur = 0, f_next = 0, fv_next2 = 0;
    if (DENSE && n_lo < n_tiles) {
        if (p.mask_flags) {
            f_cur = __builtin_amdgcn_readfirstlane(tile_flag(n_lo));
            if (n_lo + 1 < n_tiles) fv_next2 = tile_flag(n_lo + 1);
        }
        if (f_cur == 0) { if (STAGED) tile_copy(n_lo); else tile_values(n_lo); }
    }
    for (int t = n_lo; t < n_tiles; ++t) {
        // Tile t has landed for everyone, tile t - 1's P and dS are in the exchange buffer, and everyone is done with tile
        // t - 2: its stage is free for tile t + 1.
        __builtin_amdgcn_s_waitcnt(0x0F70);             // vmcnt(0)
        asm volatile("" ::: "memory");
        __syncthreads();
        if (DENSE) {      // (arrived: waits the compiler places for these are placed here, before the next copies are issued)
            asm volatile("" : "+v"(fv_next2));
            f_next = t + 1 < n_tiles && p.mask_flags ? __builtin_amdgcn_readfirstlane(fv_next2) : 0;
            if (STAGED) {
                if (f_cur == 0) {      // this tile's values out of the wavefront's buffer, which the next tile's copies may then take
#pragma unroll
                    for (int r4 = 0; r4 < 4; ++r4) {
                        const short4v x = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4v __attribute__((address_space(3)))*)(smem + NS * STAGE + XCHG + wave * 2048 + m_tr + r4 * 512));
#pragma unroll
                        for (int e = 0; e < 4; ++e) mval[2 * r4 + e / 2][e % 2] = __builtin_bit_cast(T, (short)x[e]);
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) asm volatile("" : "+v"(mnext[i]));
#pragma unroll
                for (int i = 0; i < 8; ++i) mval[i] = __builtin_bit_cast(vec2, mnext[2 * i] | (mnext[2 * i + 1] << 16));
            }
        }
        const int nstage = stage == 2 ? 0 : stage + 1;
        if (t + 1 < n_tiles) issue(nstage);
        if (DENSE) {
            if (p.mask_flags && t + 2 < n_tiles) fv_next2 = tile_flag(t + 2);
            if (t + 1 < n_tiles && f_next == 0) {
                if (STAGED) {
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");      // (the reads above have delivered: the buffer is free)
                    tile_copy(t + 1);
                } else
                    tile_values(t + 1);
            }
        }
        // Every wavefront computes every tile: one whose keys no row of the tile sees (the first tile or two under a
        // causal mask) works on -inf, and would wait at the barriers for the others anyway.
        step(stage, pstage, i0, t > n_lo, f_cur, std::true_type{});
        pstage = stage;
        stage = nstage;
        i0 = i0 + PF_BN >= n_qt * PF_BN ? t_begin * PF_BN : i0 + PF_BN;      // (then: next head of the group)
        f_cur = f_next;
    }
    if (n_lo < n_tiles) {
        __syncthreads();
        step(stage, pstage, i0, true, 0, std::false_type{});
    }

    if (parts > 1) {
        // this stretch's sums as f32 into its plane of the workspace (contiguous rows of D and Dv floats); the pass behind
        // the kernel adds the planes in order and writes the gradients' rows
        if (my_j < Skv) {
            const int64_t r = (((int64_t)part * p.B + b) * p.Hkv + hkv) * Skv + my_j;
            float* krow = bp.part_dk + r * p.D + role * (D / 2);
            float* vrow = bp.part_dv + r * p.Dv + role * (D / 2);
#pragma unroll
            for (int d = 0; d < NCB; ++d)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    float4v wk, wv;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        wk[e] = my_j < kv_len ? dk_acc[d][r4 * 4 + e] * p.scale : 0.0f;
                        wv[e] = my_j < kv_len ? dv_acc[d][r4 * 4 + e] : 0.0f;
                    }
                    const int col = role * (D / 2) + d * 32 + r4 * 8 + g * 4;
                    if (col < p.D) *(float4v*)(krow + d * 32 + r4 * 8 + g * 4) = wk;
                    if (col < p.Dv) *(float4v*)(vrow + d * 32 + r4 * 8 + g * 4) = wv;
                }
        }
        return;
    }
    if (my_j < Skv) {
        T* krow = dkp + (int64_t)my_j * bp.dk_ss + role * (D / 2);
        T* vrow = dvp + (int64_t)my_j * bp.dv_ss + role * (D / 2);
#pragma unroll
        for (int d = 0; d < NCB; ++d)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                typedef T vec4 __attribute__((ext_vector_type(4)));
                vec4 wk, wv;
#pragma unroll
                for (int e = 0; e < 4; ++e) {       // (a key past kv_len met no mask above: its sums are not gradients)
                    wk[e] = (T)(my_j < kv_len ? dk_acc[d][r4 * 4 + e] * p.scale : 0.0f);
                    wv[e] = (T)(my_j < kv_len ? dv_acc[d][r4 * 4 + e] : 0.0f);
                }
                const int col = role * (D / 2) + d * 32 + r4 * 8 + g * 4;
                if (col < p.D) *(vec4*)(krow + d * 32 + r4 * 8 + g * 4) = wk;
                if (col < p.Dv) *(vec4*)(vrow + d * 32 + r4 * 8 + g * 4) = wv;
            }
    }
#endif
}

// dst rows [B, H, S, D] of T by strides = the sum of planes 0 .. nplanes - 1 of src ([nplanes][B, H, S, D] f32, contiguous), added
// in that order; blockIdx.y picks one of two such jobs (dK and dV share a launch).  A thread takes four elements.
template <typename T> struct SumPlanesJob {
    T* dst;
    const float* src;
    int64_t sb, sh, ss;
    int B, H, S, D;
};
template <typename T>
__global__ __launch_bounds__(256) void sdpa_bwd_sum_planes_kernel(SumPlanesJob<T> j0, SumPlanesJob<T> j1, int nplanes)
{
    typedef float float4v __attribute__((ext_vector_type(4)));
    const SumPlanesJob<T>& j = blockIdx.y == 0 ? j0 : j1;
    const int d4 = j.D >> 2;
    const int64_t n = (int64_t)j.B * j.H * j.S * d4;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const int64_t row = idx / d4;
    const int c = (int)(idx - row * d4) * 4;
    const int s = (int)(row % j.S);
    const int64_t bh = row / j.S;
    const int h = (int)(bh % j.H);
    const int64_t b = bh / j.H;
    const int64_t plane = (int64_t)j.B * j.H * j.S * j.D;
    float4v acc = *(const float4v*)(j.src + row * j.D + c);
    for (int k = 1; k < nplanes; ++k) {
        const float4v x = *(const float4v*)(j.src + k * plane + row * j.D + c);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] += x[e];
    }
    typedef T vec4 __attribute__((ext_vector_type(4)));
    vec4 w;
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = (T)acc[e];
    *(vec4*)(j.dst + b * j.sb + h * j.sh + (int64_t)s * j.ss + c) = w;
}

// The dQ kernel goes to a side stream where one is to be had (side_stream.h) - it and the dK/dV kernel read the same inputs
// and the row dots, and write different outputs - when the call is short of work: at most two rounds of dQ workgroups (two
// per compute unit at a time), or D = 64.  Measured, whole call, forked against one stream (bf16, causal): 8 heads x 1024
// 0.80 (D = 128) / 0.91 (64), 8 heads x 8192 0.875 / 0.98, 32 heads x 2048 0.98 / 0.89, 128 heads x 4096 1.00 - 1.03 / 0.96,
// 32 heads x 8192 1.01 / 0.94: at D = 128 two launches that each fill the device only disturb each other's longest-first
// order, at D = 64 the dQ kernel's workgroups still fill the dK/dV kernel's tail.  (The fork and join cost about 5 us: 32
// heads x 1024, 256 workgroups in a call of 52 - 74 us, is 8 - 9 % slower forked.)
template <typename T, int D, bool DENSE = false>
static hipError_t launch_bwd_t(const SdpaBwdParams& bp, hipStream_t stream)
{
    const SdpaParams& p = bp.f;
    const int64_t rows = (int64_t)p.B * p.Hq * p.Sq;
    const int nkb = (p.Skv + BWD_KEYS - 1) / BWD_KEYS;
    const bool with_dkv = (int64_t)nkb * p.Hkv * p.B > 0;
    const int64_t dq_total = (int64_t)((p.Sq + PF_BM - 1) / PF_BM) * p.Hq * p.B;
    SideStreamLease side(stream, rows > 0 && with_dkv && (D == 64 || dq_total <= 4 * (int64_t)device_cus()));
    bool forked = false;
    if (rows > 0) {
        hipLaunchKernelGGL((sdpa_bwd_delta_kernel<T>), dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, stream, bp);
        forked = with_dkv && side.active() && side.fork() == hipSuccess;
    }
    if (with_dkv) {
        const unsigned parts = bp.parts_kv > 1 ? (unsigned)bp.parts_kv : 1u;
        const dim3 grid((unsigned)((int64_t)nkb * p.Hkv * p.B), parts);
        if (DENSE && p.mask_chunks) hipLaunchKernelGGL((sdpa_bwd_dkv_kernel<T, D, DENSE ? 2 : 0>), grid, dim3(512), 0, stream, bp);
        else hipLaunchKernelGGL((sdpa_bwd_dkv_kernel<T, D, DENSE ? 1 : 0>), grid, dim3(512), 0, stream, bp);
        if (parts > 1) {
            const SumPlanesJob<T> jk = {(T*)bp.d_k, bp.part_dk, bp.dk_sb, bp.dk_sh, bp.dk_ss, p.B, p.Hkv, p.Skv, p.D};
            const SumPlanesJob<T> jv = {(T*)bp.d_v, bp.part_dv, bp.dv_sb, bp.dv_sh, bp.dv_ss, p.B, p.Hkv, p.Skv, p.Dv};
            const int64_t n4 = (int64_t)p.B * p.Hkv * p.Skv * (max(p.D, p.Dv) >> 2);
            hipLaunchKernelGGL((sdpa_bwd_sum_planes_kernel<T>), dim3((unsigned)((n4 + 255) / 256), 2), dim3(256), 0, stream, jk, jv, (int)parts);
        }
    }
    if (rows > 0) {
        hipStream_t sq = forked ? side.stream() : stream;
        const int nqb = (p.Sq + PF_BM - 1) / PF_BM;
        const int64_t total = (int64_t)nqb * p.Hq * p.B;
        SdpaBwdParams bq = bp;      // two workgroups per CU, an eighth of the CUs per XCD
        bq.f.interleave = work_interleave(p.causal != 0 || p.mask != nullptr, 2 * device_cus() / 8, p.G, nqb, (total & 7) == 0 ? total >> 3 : total);
        bq.f.deal_groups = (total & 7) == 0 ? work_deal(bq.f.interleave, p.G, nqb, total >> 3, p.causal != 0 || p.mask != nullptr) : 0;
        if (DENSE && p.mask_chunks) hipLaunchKernelGGL((sdpa_bwd_dq_kernel<T, D, DENSE ? 2 : 0>), dim3((unsigned)total), dim3(256), 0, sq, bq);
        else hipLaunchKernelGGL((sdpa_bwd_dq_kernel<T, D, DENSE ? 1 : 0>), dim3((unsigned)total), dim3(256), 0, sq, bq);
    }
    const hipError_t launched = hipGetLastError();
    if (forked) {
        const hipError_t e = side.join();      // (also after a failed launch: whatever did reach the side stream is ordered before the caller's next work)
        if (e != hipSuccess) return e;
    }
    return launched;
}

// Host has validated: dtype f16/bf16, D and Dv <= 128 in whole 16-byte vectors (bp.f.Dp = the instance: 64 or 128; smaller
// or unequal head dimensions are zero-padded on the way into LDS and registers, stores are cut), a dense mask of any strides (the DENSE instances), unit last-axis strides, 16-byte aligned rows,
// row strides below 2^24 elements, lse and the delta workspace present.
hipError_t launch_sdpa_bwd_mfma(const SdpaBwdParams& bp, int dtype, hipStream_t stream)
{
    if (bp.f.mask) {
        if (bp.f.Dp == 128) return dtype == 1 ? launch_bwd_t<f16_t, 128, true>(bp, stream) : launch_bwd_t<bf16_t, 128, true>(bp, stream);
        return dtype == 1 ? launch_bwd_t<f16_t, 64, true>(bp, stream) : launch_bwd_t<bf16_t, 64, true>(bp, stream);
    }
    if (bp.f.Dp == 128) return dtype == 1 ? launch_bwd_t<f16_t, 128>(bp, stream) : launch_bwd_t<bf16_t, 128>(bp, stream);
    return dtype == 1 ? launch_bwd_t<f16_t, 64>(bp, stream) : launch_bwd_t<bf16_t, 64>(bp, stream);
}

}  // namespace incin_rocm
