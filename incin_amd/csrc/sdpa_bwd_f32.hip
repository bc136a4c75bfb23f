// f32 attention backward on the gfx950 matrix cores with IEEE single-precision arithmetic (v_mfma_f32_32x32x2_f32),
// D == Dv in {64, 128}: dQ, dK, dV of O = softmax(Q K^T s + mask) V for an upstream gradient dO, from Q, K, V, O, dO
// and the forward's row normalisers L_i.  f32 is the dtype the reference trains in; its gradient is what walking the
// tape of the composed ops gives (crates/incin-backends/src/cpu/ops/shape_ops.rs:1245-1269, cpu/tape.rs:149-176).
//
//   P_ij = exp(x_ij - L_i)      dP_ij = dO_i . V_j      D_i = dO_i . O_i      dS_ij = P_ij (dP_ij - D_i)
//   dV_j = sum_i P_ij dO_i      dK_j = s sum_i dS_ij Q_i      dQ_i = s sum_j dS_ij K_j
//
// Three kernels, no atomics (results are the same on every run), P and dP recomputed in both big ones - the plan of
// sdpa_bwd_mfma.hip with the operand layouts of sdpa_prefill_f32.hip:
//   bwd_f32_delta_kernel   per query row, into the workspace: -L_i log2(e) and -D_i, the values both big kernels start
//                          their S and dP accumulators from
//   bwd_f32_dq_kernel      the forward's shape of work: a wavefront owns 32 query rows (Q' and dO rows resident as B
//                          operands), K / V tiles stream through LDS; S^T = K Q'^T and dP^T = V dO^T land in the
//                          lane-owns-a-query layout, which is the B-operand layout of dQ^T += K^T dS^T (K^T read from
//                          the K tile as 32 consecutive floats of one row per half-wavefront)
//   bwd_f32_dkv_kernel     the roles swapped: a wavefront owns 32 keys (K' and V rows resident as B operands), Q / dO
//                          tiles of the group's query heads stream through LDS; S = Q K'^T and dP = dO V^T land in a
//                          lane-owns-a-key layout, the B-operand layout of dV^T += dO^T P and dK^T += Q^T dS
// A matrix instruction occupies its pipe for 64 cycles and takes one register per operand, so nothing else is near a
// limit and the loops are plain.  At D = 128 the resident rows and the accumulators of a wavefront exceed 256
// registers: those instances run one wavefront per SIMD.
#include <type_traits>

#include "sdpa_bwd.h"
#include "sdpa_mfma_common.h"
#include "side_stream.h"

namespace incin_rocm {

typedef float float4v __attribute__((ext_vector_type(4)));

// The LDS tile layout of sdpa_prefill_f32.hip: 16 KiB tiles of unpadded rows, 16-byte chunks XOR-swizzled by f(row).
template <int D> struct F32Tile {
    static constexpr int ROWB = D * 4, CPR = D / 4, TILE_BYTES = 16384;
    static constexpr int ROWS = TILE_BYTES / ROWB;           // 64 (D = 64), 32 (D = 128)
    static constexpr int NB = ROWS / 32, LPW = TILE_BYTES / 1024 / 4;
    static __device__ __forceinline__ int f(int r) { return (r & 3) | ((r & 4) << 1) | ((r & 8) >> 1); }
};

// Per-lane addressing of a tile, for both ways a tile is read: by rows (lane (ql, g): 16 bytes of row ql, floats
// 8 j + 4 g ..: an A operand whose M index is the row) and by columns (lane (ql, g), k-step r: float 32 db + ql of row
// 8 (r / 4) + 4 g + r % 4: an A operand whose M index is the column), and of the global -> LDS copies.
template <int D> struct F32Addr {
    typedef F32Tile<D> L;
    int row_base;                  // by rows: address = row_base ^ (j << 5)
    int col_low[8], col_high[D / 32];
    int voff[2][L::LPW];
    int width[2];                  // [tensor]: floats of data per row (a row's chunks beyond arrive as zeros: dma_chunk_offset)

    __device__ __forceinline__ void init(int wave, int lane, int64_t stride0, int64_t stride1, int width0, int width1)
    {
        width[0] = width0;
        width[1] = width1;
        const int ql = lane & 31, g = lane >> 5;
        row_base = ql * L::ROWB + (((g ^ L::f(ql)) & 1) << 4) + ((L::f(ql) & 0xe) << 4);
#pragma unroll
        for (int c = 0; c < 8; ++c) col_low[c] = 4 * g * L::ROWB + (((ql >> 2) ^ c) << 4) + (ql & 3) * 4;
#pragma unroll
        for (int db = 0; db < D / 32; ++db) col_high[db] = (db ^ g) << 7;
#pragma unroll
        for (int c = 0; c < L::LPW; ++c) {
            const int pos = (wave * L::LPW + c) * 64 + lane;
            const int row = pos / L::CPR, slot = pos % L::CPR;
            voff[0][c] = dma_chunk_offset(row, (int)stride0 * 4, slot ^ L::f(row), width0 * 4);
            voff[1][c] = dma_chunk_offset(row, (int)stride1 * 4, slot ^ L::f(row), width1 * 4);
        }
    }
    __device__ __forceinline__ float4v by_rows(const char* tile, int blk, int j) const
    {
        return *(const float4v*)(tile + blk * 32 * L::ROWB + (row_base ^ (j << 5)));
    }
    __device__ __forceinline__ float by_cols(const char* tile, int blk, int r, int db) const
    {
        return *(const float*)(tile + (blk * 32 + (r / 8) * 16 + 8 * ((r / 4) % 2) + r % 4) * L::ROWB + col_low[(r % 4) | (4 * ((r / 4) % 2))] + col_high[db]);
    }
    // rows [row0, row0 + ROWS) of tensor `which` (rows of `stride` floats, `rows` of them) into the tile at LDS address dst
    __device__ __forceinline__ void issue(int which, const float* base, int64_t stride, int rows, int row0, unsigned dst, int wave) const
    {
        int64_t rem = (int64_t)(rows - row0 - 1) * stride * 4 + width[which] * 4;
        if (rem > 0x7fffffffLL) rem = 0x7fffffffLL;
        if (rem < 0) rem = 0;
        const uint4v r = dma_descriptor((const char*)base + (int64_t)row0 * stride * 4, (int)rem);
#pragma unroll
        for (int c = 0; c < L::LPW; ++c) dma_copy16(r, dst + (wave * L::LPW + c) * 1024, voff[which][c]);
    }
};

// ---- -L_i log2(e) and -D_i ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void bwd_f32_delta_kernel(SdpaBwdParams p)
{
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);     // (b * Hq + hq) * Sq + i
    const int64_t rows = (int64_t)p.f.B * p.f.Hq * p.f.Sq;
    if (row >= rows) return;
    const int i = (int)(row % p.f.Sq);
    const int64_t bh = row / p.f.Sq;
    const int hq = (int)(bh % p.f.Hq), b = (int)(bh / p.f.Hq);
    const float* o = (const float*)p.f.o + b * p.f.o_sb + hq * p.f.o_sh + (int64_t)i * p.f.o_ss;
    const float* g = (const float*)p.d_o + b * p.do_sb + hq * p.do_sh + (int64_t)i * p.do_ss;
    float acc = 0.0f;
    for (int d = lane; d < p.f.Dv; d += 64) acc = fmaf(o[d], g[d], acc);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane == 0) {
        // a row without a visible key (L_i = -inf, O and so D_i NaN) gets -inf and 0: its P is then 0 everywhere
        const float l = p.f.lse[row];
        p.neg_delta[row] = l == -INFINITY ? 0.0f : -acc;
        p.neg_l2[row] = l == -INFINITY ? -INFINITY : -l * 1.4426950408889634f;
    }
}

// ---- dQ ----------------------------------------------------------------------------------------------------------------
// DENSE: a dense additive mask - its values (times log2 e) are added to the scores before the exponential; what it hides
// (-inf) ends as P = 0 like the causal edge.  A lane owns a query: the 16 keys of a block are four 16-byte loads of its row
// of the mask, asked for one tile ahead (right after the next tile's copies are issued) so that they arrive with that
// tile.  The mask's block flags (mask_classify_kernel ran before) give the first and the last tile in which any row of the
// workgroup sees a key: the tiles outside are left out.
template <int D, bool DENSE = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(D == 128 ? 1 : 2, D == 128 ? 1 : 2)))
void bwd_f32_dq_kernel(SdpaBwdParams bp)
{
#if defined(__HIP_DEVICE_COMPILE__)
    typedef F32Tile<D> L;
    constexpr int NJ = D / 8, NDB = D / 32, KT = L::ROWS, NB = L::NB;
    const SdpaParams& p = bp.f;
    __shared__ __attribute__((aligned(1024))) char smem[4 * L::TILE_BYTES];      // K buffers 0, 1, V buffers 0, 1

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ql = lane & 31, g = lane >> 5;
    const int Sq = p.Sq, Skv = p.Skv;
    const int nqb = (Sq + PF_BM - 1) / PF_BM;
    const int total = gridDim.x;
    const WorkItem wi = (total & 7) == 0 ? work_item_of_share(blockIdx.x & 7, blockIdx.x >> 3, total >> 3, p.interleave, p.G, nqb, p.deal_groups)
                                         : work_item(blockIdx.x, p.interleave, p.G, nqb);
    const int hkv = wi.bhkv % p.Hkv, b = wi.bhkv / p.Hkv;
    const int hq = hkv * p.G + wi.gq;
    const int q0 = wi.qblk * PF_BM;

    const float* qp = (const float*)p.q + (int64_t)b * p.q_sb + (int64_t)hq * p.q_sh;
    const float* gp = (const float*)bp.d_o + (int64_t)b * bp.do_sb + (int64_t)hq * bp.do_sh;
    const float* kp = (const float*)p.k + (int64_t)b * p.k_sb + (int64_t)hkv * p.k_sh;
    const float* vp = (const float*)p.v + (int64_t)b * p.v_sb + (int64_t)hkv * p.v_sh;
    float* dqp = (float*)bp.d_q + (int64_t)b * bp.dq_sb + (int64_t)hq * bp.dq_sh;

    int kv_len = Skv;
    if (p.kv_lens) kv_len = clampi(p.kv_lens[b], 0, Skv);
    // query rows at and beyond rows_b are padding (q_lens): their dQ is written as zero; a lane's row stays in its own
    // column of every product here, so a padding row next to real ones computes in isolation
    const int rows_b = p.q_lens ? clampi(p.q_lens[b], 0, Sq) : Sq;
    const int coff = Skv - Sq;
    int j_end = kv_len;
    const int my_i = q0 + wave * 32 + ql;
    int lim_lane = kv_len, lim_wave_min = kv_len, lim_wave_max = kv_len;
    if (p.causal) {
        const int last_row = min(q0 + PF_BM - 1, rows_b - 1);
        j_end = clampi(last_row + coff + 1, 0, kv_len);
        lim_lane = clampi(my_i + coff + 1, 0, kv_len);
        lim_wave_min = clampi(q0 + wave * 32 + coff + 1, 0, kv_len);
        lim_wave_max = clampi(min(q0 + wave * 32 + 31, rows_b - 1) + coff + 1, 0, kv_len);
    }
    if (q0 >= rows_b) j_end = 0;
    if (q0 + wave * 32 >= rows_b) lim_wave_min = lim_wave_max = 0;
    int n_tiles = (j_end + KT - 1) / KT, t_first = 0;
    const int n_act = lim_wave_max > 0 ? (lim_wave_max + KT - 1) / KT : 0;
    if (DENSE && p.mask_flags) {
        __shared__ int s_seen[2];
        const int nkb32 = (Skv + 31) >> 5, nrb32 = (Sq + 31) >> 5;
        const uint8_t* fl = mask_flags_of(p, b, hq);
        if (tid == 0) { s_seen[0] = 0x7fffffff; s_seen[1] = -1; }
        __syncthreads();
        int lo = 0x7fffffff, hi = -1;
        for (int c = tid; c < min(NB * n_tiles, nkb32); c += 256) {
            bool seen = false;
#pragma unroll
            for (int w = 0; w < 4; ++w) seen = seen || fl[(int64_t)min((q0 >> 5) + w, nrb32 - 1) * nkb32 + c] != 2;
            if (seen) { lo = min(lo, c); hi = max(hi, c); }
        }
        if (hi >= 0) { atomicMin(&s_seen[0], lo); atomicMax(&s_seen[1], hi); }
        __syncthreads();
        t_first = s_seen[1] < 0 ? 0 : __builtin_amdgcn_readfirstlane(s_seen[0]) / NB;
        n_tiles = s_seen[1] < 0 ? 0 : min(n_tiles, __builtin_amdgcn_readfirstlane(s_seen[1]) / NB + 1);
    }

    // this workgroup's share of the tiles (bp.parts_q workgroups per block of rows: blockIdx.y says which)
    const int part = blockIdx.y;
    if (gridDim.y > 1) {
        const int span = max(n_tiles - t_first, 0), parts = gridDim.y;
        const int lo = t_first + (int)((int64_t)span * part / parts), hi = t_first + (int)((int64_t)span * (part + 1) / parts);
        t_first = lo;
        n_tiles = hi;
    }

    F32Addr<D> ad;
    ad.init(wave, lane, p.k_ss, p.v_ss, p.D, p.Dv);
    const unsigned lds0 = lds_address(smem);
    auto issue_kv = [&](int t) __attribute__((always_inline)) {
        ad.issue(0, kp, p.k_ss, j_end, t * KT, lds0 + (t & 1) * L::TILE_BYTES, wave);
        ad.issue(1, vp, p.v_ss, j_end, t * KT, lds0 + (2 + (t & 1)) * L::TILE_BYTES, wave);
    };

    // resident B operands of this lane's query: Q' = Q * scale * log2(e) (scores in log2 units) and dO
    float4v qreg[NJ], greg[NJ];
    float seed_s, seed_d;
    {
        const int qi = min(my_i, Sq - 1);
        const float* qrow = qp + (int64_t)qi * p.q_ss + g * 4;
        const float* grow = gp + (int64_t)qi * bp.do_ss + g * 4;
        const float c2 = p.scale * 1.4426950408889634f;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            // (beyond the head dimensions: zeros, like the tiles' rows)
            const bool in_q = j * 8 + g * 4 < p.D, in_g = j * 8 + g * 4 < p.Dv;
            if (in_q) qreg[j] = *(const float4v*)(qrow + j * 8);
            if (in_g) greg[j] = *(const float4v*)(grow + j * 8);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                qreg[j][e] = in_q ? qreg[j][e] * c2 : 0.0f;
                greg[j][e] = in_g ? greg[j][e] : 0.0f;
            }
        }
        const int64_t stat = ((int64_t)b * p.Hq + hq) * Sq + qi;
        seed_s = bp.neg_l2[stat];
        seed_d = bp.neg_delta[stat];
        // All of these have to have arrived before the loop: a wait the compiler places for them inside it comes after
        // the copies of the next tile were issued (which it does not know of) and, memory operations completing in
        // order, would wait for those as well - a full memory latency in every tile.
#pragma unroll
        for (int j = 0; j < NJ; ++j) asm volatile("" : "+v"(greg[j]));
        asm volatile("" : "+v"(seed_s), "+v"(seed_d));
    }
    floatx16 dq_acc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) dq_acc[db][r] = 0.0f;

    // DENSE: this lane's row of the mask; the values of a tile's keys, register r of block kb being key
    // t * KT + 32 * kb + 8 * (r / 4) + 4 * g + r % 4
    [[maybe_unused]] float4v m_next[NB][4], m_cur[NB][4];
    [[maybe_unused]] const float* mrow = nullptr;
    [[maybe_unused]] bool m_vec = false;
    if (DENSE) {
        mrow = (const float*)p.mask + (int64_t)b * p.m_sb + (int64_t)hq * p.m_sh + (int64_t)min(my_i, Sq - 1) * p.m_si;
        m_vec = p.mask_vec && (reinterpret_cast<uintptr_t>(p.mask) & 15u) == 0;
    }
    [[maybe_unused]] auto load_mask = [&](int t) __attribute__((always_inline)) {
#pragma unroll
        for (int kb = 0; kb < NB; ++kb)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const int j = t * KT + 32 * kb + 8 * r4 + 4 * g;
                if (m_vec && j + 3 < Skv) m_next[kb][r4] = *(const float4v*)(mrow + j);
                else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) m_next[kb][r4][e] = mrow[(int64_t)min(j + e, Skv - 1) * p.m_sj];
                }
            }
    };
    if (t_first < n_tiles) {
        issue_kv(t_first);
        if (DENSE) load_mask(t_first);
    }
    for (int t = t_first; t < n_tiles; ++t) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (DENSE) {      // (arrived: a wait the compiler places for them is placed here, before the next copies are issued)
#pragma unroll
            for (int kb = 0; kb < NB; ++kb)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    m_cur[kb][r4] = m_next[kb][r4];
                    asm volatile("" : "+v"(m_cur[kb][r4]));
                }
        }
        if (t + 1 < n_tiles) {
            issue_kv(t + 1);
            if (DENSE) load_mask(t + 1);
        }
        if (t >= n_act) continue;
        const char* kt = smem + (t & 1) * L::TILE_BYTES;
        const char* vt = smem + (2 + (t & 1)) * L::TILE_BYTES;
#pragma unroll
        for (int kb = 0; kb < NB; ++kb) {
            const int j0 = t * KT + kb * 32;
            if (j0 >= lim_wave_max) break;
            // S^T - L and dP^T - D: the accumulators start from the per-query values.  Operands of step j + 1 are read
            // from LDS before the matrix instructions of step j are issued (the fences keep the compiler from moving
            // the reads back down to their first use, where each would expose its latency).
            floatx16 s, dp;
#pragma unroll
            for (int r = 0; r < 16; ++r) { s[r] = seed_s; dp[r] = seed_d; }
            float4v ka = ad.by_rows(kt, kb, 0), va = ad.by_rows(vt, kb, 0);
            float kk[NDB];
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                float4v kn = ka, vn = va;
                if (j + 1 < NJ) {
                    kn = ad.by_rows(kt, kb, j + 1);
                    vn = ad.by_rows(vt, kb, j + 1);
                } else {
#pragma unroll
                    for (int db = 0; db < NDB; ++db) kk[db] = ad.by_cols(kt, kb, 0, db);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    s = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[e], qreg[j][e], s, 0, 0, 0);
                    dp = __builtin_amdgcn_mfma_f32_32x32x2f32(va[e], greg[j][e], dp, 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                ka = kn;
                va = vn;
            }
            {
                // keys at and past this lane's limit: only blocks that cross a limit of the wavefront have any
                const int rel = j0 + 32 > lim_wave_min ? lim_lane - (j0 + 4 * g) : 64;
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (8 * (r / 4) + (r % 4) >= rel) s[r] = -INFINITY;
            }
            if (DENSE) {
#pragma unroll
                for (int r = 0; r < 16; ++r) s[r] = __builtin_fmaf(m_cur[kb][r / 4][r % 4], 1.4426950408889634f, s[r]);
            }
            // dS^T = P^T (dP^T - D); a masked pair has P = 0 and a finite second factor
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] = __builtin_amdgcn_exp2f(s[r]) * dp[r];
            // dQ^T += K^T dS^T: k-step r takes keys kappa(r, 0), kappa(r, 1)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float kn[NDB];
#pragma unroll
                for (int db = 0; db < NDB; ++db) kn[db] = r + 1 < 16 ? ad.by_cols(kt, kb, r + 1, db) : 0.0f;
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int db = 0; db < NDB; ++db) dq_acc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(kk[db], s[r], dq_acc[db], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int db = 0; db < NDB; ++db) kk[db] = kn[db];
            }
        }
    }
    if (my_i < Sq) {
        float* row = dqp + (int64_t)my_i * bp.dq_ss;
        if (part > 0)      // (a plane of the workspace: contiguous rows of D floats)
            row = bp.part_dq + ((((int64_t)(part - 1) * p.B + b) * p.Hq + hq) * Sq + my_i) * p.D;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                float4v w;
#pragma unroll
                for (int e = 0; e < 4; ++e) w[e] = my_i < rows_b ? dq_acc[db][r4 * 4 + e] * p.scale : 0.0f;
                if (db * 32 + r4 * 8 + g * 4 < p.D) *(float4v*)(row + db * 32 + r4 * 8 + g * 4) = w;
            }
    }
#endif
}

// ---- dK, dV ------------------------------------------------------------------------------------------------------------
constexpr int BWD32_KEYS = 128;      // keys per workgroup: 32 per wavefront

// DENSE: a dense additive mask.  A lane owns a key and holds 16 query rows of a block: its values are 16 loads down a column
// of the mask (one buffer descriptor per tile that starts at the tile's first row and ends with the head's last - rows past
// Sq read zeros - one lane offset for the key's column and the lane's first row, a scalar offset per register; the host has
// checked that a tile's rows fit 32-bit offsets), asked for one tile ahead like the dQ kernel's.  The block flags trim the
// tiles to those between the first and the last block of rows, over the group's heads, that see any key of the workgroup.
template <int D, bool DENSE = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(D == 128 ? 1 : 2, D == 128 ? 1 : 2)))
void bwd_f32_dkv_kernel(SdpaBwdParams bp)
{
#if defined(__HIP_DEVICE_COMPILE__)
    typedef F32Tile<D> L;
    constexpr int NJ = D / 8, NDB = D / 32, QT = L::ROWS, NB = L::NB;
    constexpr int STAGE = 2 * L::TILE_BYTES + 1024;          // Q tile, dO tile, the two per-row arrays of the tile
    const SdpaParams& p = bp.f;
    __shared__ __attribute__((aligned(1024))) char smem[2 * STAGE];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ql = lane & 31, g = lane >> 5;
    const int Sq = p.Sq, Skv = p.Skv;
    const int nkb = (Skv + BWD32_KEYS - 1) / BWD32_KEYS;
    // all key blocks of a (batch, KV head) pair read the same Q and dO rows: a pair is given to one XCD
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
    const int j0 = kblk * BWD32_KEYS;
    const int my_j = j0 + wave * 32 + ql;              // this lane's key

    const float* kp = (const float*)p.k + (int64_t)b * p.k_sb + (int64_t)hkv * p.k_sh;
    const float* vp = (const float*)p.v + (int64_t)b * p.v_sb + (int64_t)hkv * p.v_sh;
    float* dkp = (float*)bp.d_k + (int64_t)b * bp.dk_sb + (int64_t)hkv * bp.dk_sh;
    float* dvp = (float*)bp.d_v + (int64_t)b * bp.dv_sb + (int64_t)hkv * bp.dv_sh;

    int kv_len = Skv;
    if (p.kv_lens) kv_len = clampi(p.kv_lens[b], 0, Skv);
    const int coff = Skv - Sq;
    // query rows that see any key of this workgroup: i >= j - coff for its first key (causal)
    const int i_begin_wg = p.causal ? clampi(j0 - coff, 0, Sq) : 0;
    // first query row that sees every key of this wavefront: tiles from there on need no mask
    const int i_all_wave = p.causal ? max(j0 + wave * 32 + 31 - coff, 0) : 0;
    int t_begin = i_begin_wg / QT;
    // query rows at and beyond rows_b are padding (q_lens): the tiles end there, and the rows between there and the end of
    // the last tile arrive as zeros like rows past Sq
    const int rows_b = p.q_lens ? clampi(p.q_lens[b], 0, Sq) : Sq;
    int n_qt = (rows_b + QT - 1) / QT;
    if (DENSE && p.mask_flags) {
        __shared__ int s_seen[2];
        const int nkb32 = (Skv + 31) >> 5, nrb32 = (Sq + 31) >> 5, c0 = kblk * 4;
        if (tid == 0) { s_seen[0] = 0x7fffffff; s_seen[1] = -1; }
        __syncthreads();
        int lo = 0x7fffffff, hi = -1;
        const int r_lo = NB * t_begin, r_n = min(NB * n_qt, nrb32) - r_lo;
        for (int x = tid; x < r_n * p.G; x += 256) {
            const int rb = r_lo + x % r_n;
            const uint8_t* fl = mask_flags_of(p, b, hkv * p.G + x / r_n) + (int64_t)rb * nkb32;
            bool seen = false;
#pragma unroll
            for (int c = 0; c < 4; ++c) seen = seen || fl[min(c0 + c, nkb32 - 1)] != 2;
            if (seen) { lo = min(lo, rb); hi = max(hi, rb); }
        }
        if (hi >= 0) { atomicMin(&s_seen[0], lo); atomicMax(&s_seen[1], hi); }
        __syncthreads();
        if (s_seen[1] < 0) n_qt = t_begin;
        else {
            t_begin = __builtin_amdgcn_readfirstlane(s_seen[0]) / NB;
            n_qt = __builtin_amdgcn_readfirstlane(s_seen[1]) / NB + 1;
        }
    }
    const int tiles_per_head = j0 < kv_len ? max(n_qt - t_begin, 0) : 0;
    const int n_all = tiles_per_head * p.G;             // the group's query heads one after another
    // this workgroup's share of the walk (bp.parts_kv workgroups per key block: blockIdx.y says which)
    const int part = blockIdx.y;
    const int n_lo = (int)((int64_t)n_all * part / (int)gridDim.y), n_tiles = (int)((int64_t)n_all * (part + 1) / (int)gridDim.y);

    F32Addr<D> ad;
    ad.init(wave, lane, p.q_ss, bp.do_ss, p.D, p.Dv);

    // this lane's key: K' = K * scale * log2(e) and V rows as B operands
    float4v kreg[NJ], vreg[NJ];
    {
        const int kj = clampi(my_j, 0, max(kv_len, 1) - 1);      // (rows past the batch entry's key count are never read)
        const float* krow = kp + (int64_t)kj * p.k_ss + g * 4;
        const float* vrow = vp + (int64_t)kj * p.v_ss + g * 4;
        const float c2 = p.scale * 1.4426950408889634f;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const bool in_k = j * 8 + g * 4 < p.D, in_v = j * 8 + g * 4 < p.Dv;
            if (in_k) kreg[j] = *(const float4v*)(krow + j * 8);
            if (in_v) vreg[j] = *(const float4v*)(vrow + j * 8);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                kreg[j][e] = in_k ? kreg[j][e] * c2 : 0.0f;
                vreg[j][e] = in_v ? vreg[j][e] : 0.0f;
            }
        }
        // (arrived before the loop, as in the dQ kernel)
#pragma unroll
        for (int j = 0; j < NJ; ++j) asm volatile("" : "+v"(vreg[j]));
    }
    // rows i >= lo_i see this lane's key under the causal mask
    const int lo_i = p.causal ? my_j - coff : -0x40000000;

    floatx16 dk_acc[NDB], dv_acc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) { dk_acc[db][r] = 0.0f; dv_acc[db][r] = 0.0f; }

    const unsigned lds0 = lds_address(smem);
    // tile `n` of the walk over (head of the group, query tile): its Q rows, dO rows and the two per-row arrays
    auto issue = [&](int n, int stage) __attribute__((always_inline)) {
        const int h = n / tiles_per_head, r0 = (t_begin + n % tiles_per_head) * QT;
        const int hq = hkv * p.G + h;
        const unsigned st = lds0 + stage * STAGE;
        ad.issue(0, (const float*)p.q + (int64_t)b * p.q_sb + (int64_t)hq * p.q_sh, p.q_ss, rows_b, r0, st, wave);
        ad.issue(1, (const float*)bp.d_o + (int64_t)b * bp.do_sb + (int64_t)hq * bp.do_sh, bp.do_ss, rows_b, r0, st + L::TILE_BYTES, wave);
        if (wave < 2) {          // 64 floats (a tile has at most that many rows) of one of the two per-row arrays; rows past Sq arrive as zeros
            const float* src = (wave == 0 ? bp.neg_l2 : bp.neg_delta) + ((int64_t)b * p.Hq + hq) * Sq + r0;
            dma_copy4(dma_descriptor(src, (rows_b - r0) * 4), st + 2 * L::TILE_BYTES + wave * 256, lane * 4);
        }
    };

    // DENSE: the mask's values of a tile, register r of block qb being query row r0 + 32 * qb + 8 * (r / 4) + 4 * g + r % 4
    [[maybe_unused]] float m_next[NB][16], m_cur[NB][16];
    [[maybe_unused]] const int m_lane = (int)(((int64_t)min(my_j, Skv - 1) * p.m_sj + (int64_t)(4 * g) * p.m_si) * 4);
    [[maybe_unused]] const int m_row4 = (int)(p.m_si * 4);
    [[maybe_unused]] auto load_mask = [&](int n) __attribute__((always_inline)) {
        const int h = n / tiles_per_head, r0 = (t_begin + n % tiles_per_head) * QT;
        const float* mc = (const float*)p.mask + (int64_t)b * p.m_sb + (int64_t)(hkv * p.G + h) * p.m_sh + (int64_t)r0 * p.m_si;
        const int64_t left = r0 < Sq ? ((int64_t)(Sq - 1 - r0) * p.m_si + (int64_t)(Skv - 1) * p.m_sj + 1) * 4 : 0;
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)mc, 0, (int)min(left, (int64_t)0x7fffffff), 0x00020000);
#pragma unroll
        for (int qb = 0; qb < NB; ++qb)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                m_next[qb][r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs, m_lane, (32 * qb + 8 * (r / 4) + (r % 4)) * m_row4, 0));
    };
    if (n_lo < n_tiles) {
        issue(n_lo, n_lo & 1);
        if (DENSE) load_mask(n_lo);
    }
    for (int n = n_lo; n < n_tiles; ++n) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (DENSE) {      // (arrived: a wait the compiler places for them is placed here, before the next copies are issued)
#pragma unroll
            for (int qb = 0; qb < NB; ++qb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    m_cur[qb][r] = m_next[qb][r];
                    asm volatile("" : "+v"(m_cur[qb][r]));
                }
        }
        if (n + 1 < n_tiles) {
            issue(n + 1, (n + 1) & 1);
            if (DENSE) load_mask(n + 1);
        }
        const char* qt = smem + (n & 1) * STAGE;
        const char* gt = qt + L::TILE_BYTES;
        const char* nl = gt + L::TILE_BYTES;
        const int i0 = (t_begin + n % tiles_per_head) * QT;
#pragma unroll
        for (int qb = 0; qb < NB; ++qb) {
            const int ib = i0 + qb * 32;               // first query row of the block
            if (ib >= rows_b) break;
            // S - L and dP - D in the lane-owns-a-key layout: register r is query row ib + 8 (r / 4) + 4 g + r % 4.
            // Operands of a step are read from LDS one step ahead, as in the dQ kernel.
            floatx16 s, dp;
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const float4v a = *(const float4v*)(nl + (qb * 32 + 8 * r4 + 4 * g) * 4);
                const float4v d = *(const float4v*)(nl + 256 + (qb * 32 + 8 * r4 + 4 * g) * 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) { s[4 * r4 + e] = a[e]; dp[4 * r4 + e] = d[e]; }
            }
            float4v qa = ad.by_rows(qt, qb, 0), ga = ad.by_rows(gt, qb, 0);
            float gg[NDB], qq[NDB];
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                float4v qn = qa, gn = ga;
                if (j + 1 < NJ) {
                    qn = ad.by_rows(qt, qb, j + 1);
                    gn = ad.by_rows(gt, qb, j + 1);
                } else {
#pragma unroll
                    for (int db = 0; db < NDB; ++db) { gg[db] = ad.by_cols(gt, qb, 0, db); qq[db] = ad.by_cols(qt, qb, 0, db); }
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    s = __builtin_amdgcn_mfma_f32_32x32x2f32(qa[e], kreg[j][e], s, 0, 0, 0);
                    dp = __builtin_amdgcn_mfma_f32_32x32x2f32(ga[e], vreg[j][e], dp, 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                qa = qn;
                ga = gn;
            }
            {
                // rows of the block that do not see this lane's key (only blocks before i_all_wave have any)
                const int rel = ib < i_all_wave ? lo_i - ib - 4 * g : -64;
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (8 * (r / 4) + (r % 4) < rel) s[r] = -INFINITY;
            }
            if (DENSE) {
#pragma unroll
                for (int r = 0; r < 16; ++r) s[r] = __builtin_fmaf(m_cur[qb][r], 1.4426950408889634f, s[r]);
            }
            // rows past Sq arrive as zeros throughout (L' = 0, dO = 0: P = exp2(q.k) finite times dP = 0 for dS, and their
            // P meets dO = 0 in dV); rows without any visible key carry -inf already
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                s[r] = __builtin_amdgcn_exp2f(s[r]);          // P
                dp[r] = s[r] * dp[r];                         // dS
            }
            // dV^T += dO^T P and dK^T += Q^T dS: k-step r takes query rows kappa(r, 0), kappa(r, 1)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float gn[NDB], qn[NDB];
#pragma unroll
                for (int db = 0; db < NDB; ++db) {
                    gn[db] = r + 1 < 16 ? ad.by_cols(gt, qb, r + 1, db) : 0.0f;
                    qn[db] = r + 1 < 16 ? ad.by_cols(qt, qb, r + 1, db) : 0.0f;
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int db = 0; db < NDB; ++db) {
                    dv_acc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(gg[db], s[r], dv_acc[db], 0, 0, 0);
                    dk_acc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(qq[db], dp[r], dk_acc[db], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int db = 0; db < NDB; ++db) { gg[db] = gn[db]; qq[db] = qn[db]; }
            }
        }
    }

    if (my_j < Skv) {
        float* krow = dkp + (int64_t)my_j * bp.dk_ss;
        float* vrow = dvp + (int64_t)my_j * bp.dv_ss;
        if (part > 0) {      // (planes of the workspace: contiguous rows of D and Dv floats)
            const int64_t r = (((int64_t)(part - 1) * p.B + b) * p.Hkv + hkv) * Skv + my_j;
            krow = bp.part_dk + r * p.D;
            vrow = bp.part_dv + r * p.Dv;
        }
        const bool live = my_j < kv_len;               // (a key past kv_len met no mask above: its sums are not gradients)
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                float4v wk, wv;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    wk[e] = live ? dk_acc[db][r4 * 4 + e] * p.scale : 0.0f;
                    wv[e] = live ? dv_acc[db][r4 * 4 + e] : 0.0f;
                }
                if (db * 32 + r4 * 8 + g * 4 < p.D) *(float4v*)(krow + db * 32 + r4 * 8 + g * 4) = wk;
                if (db * 32 + r4 * 8 + g * 4 < p.Dv) *(float4v*)(vrow + db * 32 + r4 * 8 + g * 4) = wv;
            }
    }
#endif
}

// dst rows [B, H, S, D] by strides += planes 0 .. nplanes - 1 of src ([nplanes][B, H, S, D] contiguous), in that order; blockIdx.y
// picks one of two such jobs (dK and dV share a launch).  A thread takes four floats.
struct AddPlanesJob {
    float* dst;
    const float* src;
    int64_t sb, sh, ss;
    int B, H, S, D;
};
__global__ __launch_bounds__(256) void bwd_f32_add_planes_kernel(AddPlanesJob j0, AddPlanesJob j1, int nplanes)
{
    const AddPlanesJob& j = blockIdx.y == 0 ? j0 : j1;
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
    float* d = j.dst + b * j.sb + h * j.sh + (int64_t)s * j.ss + c;
    float4v acc = *(const float4v*)d;
    const int64_t plane = (int64_t)j.B * j.H * j.S * j.D;
    for (int k = 0; k < nplanes; ++k) {
        const float4v x = *(const float4v*)(j.src + k * plane + row * j.D + c);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] += x[e];
    }
    *(float4v*)d = acc;
}

template <int D, bool DENSE = false>
static hipError_t launch_bwd_f32_t(const SdpaBwdParams& bp, hipStream_t stream)
{
    const SdpaParams& p = bp.f;
    const int64_t rows = (int64_t)p.B * p.Hq * p.Sq;
    const int nqb = (p.Sq + PF_BM - 1) / PF_BM;
    const int64_t total = (int64_t)nqb * p.Hq * p.B;
    if (total > 0x7fffffffLL) return hipErrorInvalidValue;
    const int nkb = (p.Skv + BWD32_KEYS - 1) / BWD32_KEYS;
    const bool with_dkv = (int64_t)nkb * p.Hkv * p.B > 0;
    // the dQ kernel on a side stream where one is to be had (side_stream.h) - it and the dK/dV kernel read the same inputs and
    // the row dots, and write different outputs - when the call is short of work: at most two rounds of dQ workgroups (one
    // per compute unit at a time at D = 128, two at 64).  Measured, whole call, forked against one stream (causal): 8 heads x
    // 1024 0.60 (D = 128) / 0.76 (64), 32 heads x 1024 0.82 / 0.97, 32 heads x 2048 0.87 / 0.71, 8 heads x 8192 1.03 / 0.73; with
    // more work than that 0.95 - 1.06 (128 heads x 2048 0.95 / 1.02, 64 heads x 4096 without a mask 1.02 / 1.06): not forked.
    SideStreamLease side(stream, rows > 0 && with_dkv && total <= 2 * (int64_t)(D == 128 ? 1 : 2) * device_cus());
    bool forked = false;
    if (rows > 0) {
        hipLaunchKernelGGL(bwd_f32_delta_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, bp);
        forked = with_dkv && side.active() && side.fork() == hipSuccess;
    }
    const unsigned parts_q = bp.parts_q > 1 ? (unsigned)bp.parts_q : 1u, parts_kv = bp.parts_kv > 1 ? (unsigned)bp.parts_kv : 1u;
    if (with_dkv) {
        const unsigned parts = parts_kv;
        hipLaunchKernelGGL((bwd_f32_dkv_kernel<D, DENSE>), dim3((unsigned)((int64_t)nkb * p.Hkv * p.B), parts), dim3(256), 0, stream, bp);
        if (parts > 1) {
            const AddPlanesJob jk = {(float*)bp.d_k, bp.part_dk, bp.dk_sb, bp.dk_sh, bp.dk_ss, p.B, p.Hkv, p.Skv, p.D};
            const AddPlanesJob jv = {(float*)bp.d_v, bp.part_dv, bp.dv_sb, bp.dv_sh, bp.dv_ss, p.B, p.Hkv, p.Skv, p.Dv};
            const int64_t n4 = (int64_t)p.B * p.Hkv * p.Skv * (max(p.D, p.Dv) >> 2);
            hipLaunchKernelGGL(bwd_f32_add_planes_kernel, dim3((unsigned)((n4 + 255) / 256), 2), dim3(256), 0, stream, jk, jv, (int)parts - 1);
        }
    }
    if (rows > 0) {
        hipStream_t sq = forked ? side.stream() : stream;
        const unsigned parts = parts_q;
        SdpaBwdParams bq = bp;
        bq.f.interleave = work_interleave(p.causal != 0 || p.mask != nullptr, (D == 128 ? 1 : 2) * device_cus() / 8, p.G, nqb, (total & 7) == 0 ? total >> 3 : total);
        bq.f.deal_groups = (total & 7) == 0 ? work_deal(bq.f.interleave, p.G, nqb, total >> 3, p.causal != 0 || p.mask != nullptr) : 0;
        hipLaunchKernelGGL((bwd_f32_dq_kernel<D, DENSE>), dim3((unsigned)total, parts), dim3(256), 0, sq, bq);
        if (parts > 1) {
            const AddPlanesJob jq = {(float*)bp.d_q, bp.part_dq, bp.dq_sb, bp.dq_sh, bp.dq_ss, p.B, p.Hq, p.Sq, p.D};
            const int64_t n4 = (int64_t)p.B * p.Hq * p.Sq * (p.D >> 2);
            hipLaunchKernelGGL(bwd_f32_add_planes_kernel, dim3((unsigned)((n4 + 255) / 256), 1), dim3(256), 0, sq, jq, jq, (int)parts - 1);
        }
    }
    const hipError_t launched = hipGetLastError();
    if (forked) {
        const hipError_t e = side.join();      // (also after a failed launch: whatever did reach the side stream is ordered before the caller's next work)
        if (e != hipSuccess) return e;
    }
    return launched;
}

// Host has validated: f32, D and Dv <= 128 in whole 16-byte vectors (bp.f.Dp = the instance: 64 or 128), finite scale, unit last-axis strides, 16-byte aligned rows,
// row strides below 2^22 elements, lse and the workspace present; a dense mask (the DENSE instances) of any non-negative strides
// of which 64 rows fit 32-bit byte offsets, its block flags computed.
hipError_t launch_sdpa_bwd_f32(const SdpaBwdParams& bp, hipStream_t stream)
{
    if (bp.f.mask) return bp.f.Dp == 128 ? launch_bwd_f32_t<128, true>(bp, stream) : launch_bwd_f32_t<64, true>(bp, stream);
    return bp.f.Dp == 128 ? launch_bwd_f32_t<128>(bp, stream) : launch_bwd_f32_t<64>(bp, stream);
}

}  // namespace incin_rocm
