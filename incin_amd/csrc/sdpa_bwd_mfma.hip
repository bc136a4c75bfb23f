// bf16 / f16 attention backward on the gfx950 matrix cores, head dimension 128: dQ, dK, dV of
// O = softmax(Q K^T s + mask) V for an upstream gradient dO, from Q, K, V, O, dO and the forward's row
// normalisers L_i = log sum_j exp(x_ij) (the reference reaches the same gradients by walking its tape of
// composed ops: crates/incin-backends/src/cpu/ops/matmul.rs:264-281, cpu/ops/elementwise.rs:1062-1077).
//
//   P_ij = exp(x_ij - L_i)      dP_ij = dO_i . V_j      D_i = dO_i . O_i      dS_ij = P_ij (dP_ij - D_i)
//   dV_j = sum_i P_ij dO_i      dK_j = s sum_i dS_ij Q_i      dQ_i = s sum_j dS_ij K_j
//
// Three kernels, no atomics, P and dP recomputed in both big ones:
//   sdpa_bwd_delta_kernel   D_i (f32) into the workspace
//   sdpa_bwd_dq_kernel      the forward's shape of work: a wavefront owns 32 query rows (Q and dO rows resident in
//                           registers), K / V tiles stream through LDS; S^T = K Q'^T and dP^T = V dO^T have the
//                           lane-owns-a-query accumulator layout of the forward, which is again the B-operand layout
//                           of the next product, dQ^T += K^T dS^T (K^T through the transposing LDS read)
//   sdpa_bwd_dkv_kernel     the same with the roles swapped: a wavefront owns 32 keys (K and V rows resident), Q / dO
//                           tiles of the group's query heads stream through LDS; S = Q K'^T and dP = dO V^T have a
//                           lane-owns-a-key layout, the B-operand layout of dV^T += dO^T P and dK^T += Q^T dS
// Both big kernels are plain loops (one tile at a time, operands read just ahead of use); they rely on two
// wavefronts per SIMD (dQ) or none (dK/dV, 512 registers) for overlap and are not software-pipelined.
#include <type_traits>

#include "sdpa_bwd.h"
#include "sdpa_mfma_common.h"

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
        for (int d = sub * 8; d < p.f.D; d += 128) {
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
template <typename T>
struct BwdTiles {
    typedef typename Mma<T>::vec8 vec8;
    typedef PfLayout<128> L;
    static constexpr int NSTEP = 8, NDB = 4, LPW = L::LOADS_PER_WAVE;

    int row_addr[NSTEP];           // [k-step]: byte offset of this lane's 16 bytes of row ql, chunk 2*s + g
    int tr_addr[NDB][2];           // [column block][half]: byte offset of the transposing read
    int voff[2][LPW];              // [tensor][load]: global byte offset of this lane's 16 bytes of a tile

    __device__ __forceinline__ void init(int wave, int lane, int64_t stride0, int64_t stride1)
    {
        const int ql = lane & 31, g = lane >> 5, n = lane & 15, dh = (lane >> 4) & 1;
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
            row_addr[s] = ql * L::ROWB + (((2 * s + g) ^ L::fk(ql)) << 4);
        }
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int r = 8 * h + 4 * g + (n >> 2);
                const int chunk = 4 * db + 2 * dh + ((n & 3) >> 1);
                tr_addr[db][h] = r * L::ROWB + ((chunk ^ L::fk(r)) << 4) + (n & 1) * 8;
            }
#pragma unroll
        for (int c = 0; c < LPW; ++c) {
            const int pos = (wave * LPW + c) * 64 + lane;
            const int row = pos / L::CPR, slot = pos % L::CPR;
            voff[0][c] = row * (int)stride0 * 2 + (slot ^ L::fk(row)) * 16;
            voff[1][c] = row * (int)stride1 * 2 + (slot ^ L::fk(row)) * 16;
        }
    }
    // start the copy of rows [row0, row0 + 64) of tensor `which` (base pointer of the head, `rows` rows of `stride`
    // elements) into `dst`; rows at and beyond `rows` arrive as zeros
    __device__ __forceinline__ void issue(int which, const T* base, int64_t stride, int rows, int row0, unsigned dst, int wave) const
    {
        int64_t rem = (int64_t)(rows - row0 - 1) * stride * 2 + 256;
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
    // A operand transposed: column block db (32 columns), rows 16*ks .. 16*ks + 15 of the tile in the order the
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
template <typename T>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void sdpa_bwd_dq_kernel(SdpaBwdParams bp)
{
#if defined(__HIP_DEVICE_COMPILE__)
    typedef typename Mma<T>::vec8 vec8;
    typedef PfLayout<128> L;
    constexpr int NSTEP = 8, NDB = 4, D = 128;
    const SdpaParams& p = bp.f;
    __shared__ __attribute__((aligned(1024))) char smem[4 * L::TILE_BYTES];      // K buffers 0, 1, V buffers 0, 1

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
    const int coff = Skv - Sq;
    const int my_i = q0 + wave * 32 + ql;
    int j_end = kv_len, lim_lane = kv_len, lim_wave_max = kv_len;
    if (p.causal) {
        j_end = clampi(min(q0 + PF_BM - 1, Sq - 1) + coff + 1, 0, kv_len);
        lim_lane = clampi(my_i + coff + 1, 0, kv_len);
        lim_wave_max = clampi(min(q0 + wave * 32 + 31, Sq - 1) + coff + 1, 0, kv_len);
    }
    if (q0 + wave * 32 >= Sq) lim_wave_max = 0;
    const int n_tiles = (j_end + PF_BN - 1) / PF_BN;
    const int n_act = lim_wave_max > 0 ? (lim_wave_max + PF_BN - 1) / PF_BN : 0;

    BwdTiles<T> tl;
    tl.init(wave, lane, p.k_ss, p.v_ss);

    // this lane's query: Q row (scaled into log2 units, as the forward does) and dO row, the row's normaliser and D_i
    vec8 qreg[NSTEP], greg[NSTEP];
    const int qi = min(my_i, Sq - 1);
    {
        const T* qrow = qp + (int64_t)qi * p.q_ss + g * 8;
        const T* grow = gp + (int64_t)qi * bp.do_ss + g * 8;
        const float c2 = p.scale * 1.4426950408889634f;
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
            vec8 x = *(const vec8*)(qrow + s * 16);
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = (T)((float)x[e] * c2);
            qreg[s] = x;
            greg[s] = *(const vec8*)(grow + s * 16);
        }
    }
    const int64_t stat = ((int64_t)b * p.Hq + hq) * Sq + qi;
    const float l2 = -bp.neg_l2[stat];
    const float dlt = -bp.neg_delta[stat];

    floatx16 dq_acc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) dq_acc[db][r] = 0.0f;
    floatx16 zero16;
#pragma unroll
    for (int r = 0; r < 16; ++r) zero16[r] = 0.0f;

    const unsigned lds0 = lds_address(smem);
    if (n_tiles > 0) {
        tl.issue(0, kp, p.k_ss, Skv, 0, lds0, wave);
        tl.issue(1, vp, p.v_ss, Skv, 0, lds0 + 2 * L::TILE_BYTES, wave);
    }
    for (int t = 0; t < n_tiles; ++t) {
        // K(t), V(t) have landed for everyone and everyone is done with tile t-1: the other pair of buffers is free
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (t + 1 < n_tiles) {
            tl.issue(0, kp, p.k_ss, Skv, (t + 1) * PF_BN, lds0 + ((t + 1) & 1) * L::TILE_BYTES, wave);
            tl.issue(1, vp, p.v_ss, Skv, (t + 1) * PF_BN, lds0 + (2 + ((t + 1) & 1)) * L::TILE_BYTES, wave);
        }
        if (t >= n_act) continue;
        const char* kt = smem + (t & 1) * L::TILE_BYTES;
        const char* vt = smem + (2 + (t & 1)) * L::TILE_BYTES;
        const int j0 = t * PF_BN;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            floatx16 s_acc = zero16, dp_acc = zero16;
#pragma unroll
            for (int s = 0; s < NSTEP; ++s) {
                s_acc = Mma<T>::run(tl.rows_op(kt, kb, s), qreg[s], s_acc);
                dp_acc = Mma<T>::run(tl.rows_op(vt, kb, s), greg[s], dp_acc);
            }
            // register r is key j0 + 32*kb + 8*(r/4) + 4*g + (r%4)
            vec8 ds[2];
            const int rel = lim_lane - (j0 + 32 * kb + 4 * g);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int kofs = 8 * (r / 4) + (r % 4);
                const float pr = __builtin_amdgcn_exp2f(s_acc[r] - l2);
                // (selected, not multiplied by zero: a row without visible keys has NaN in D_i and +inf here)
                ds[r / 8][r % 8] = (T)(kofs >= rel ? 0.0f : pr * (dp_acc[r] - dlt));
            }
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int db = 0; db < NDB; ++db) dq_acc[db] = Mma<T>::run(tl.tr_op(kt, db, 2 * kb + h), ds[h], dq_acc[db]);
        }
    }

    if (my_i < Sq) {
        T* row = dqp + (int64_t)my_i * bp.dq_ss;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                typedef T vec4 __attribute__((ext_vector_type(4)));
                vec4 w;
#pragma unroll
                for (int e = 0; e < 4; ++e) w[e] = (T)(dq_acc[db][r4 * 4 + e] * p.scale);
                *(vec4*)(row + db * 32 + r4 * 8 + g * 4) = w;
            }
    }
#endif
}

// ---- dK, dV ---------------------------------------------------------------------------------------------------------------
constexpr int BWD_KEYS = 128;      // keys per workgroup of the dK/dV kernel (32 per wavefront)
constexpr int BWD_RING = 8;        // matrix operands in flight from LDS (reads run this many matrix instructions ahead)

// One wavefront per SIMD, so nothing hides a latency but the wavefront's own instruction order.  A 64-query tile is
// 64 matrix instructions per wavefront in four runs of 16:
//   A0  S, dP of query rows 0-31        A1  S, dP of rows 32-63, with P and dS of rows 0-31 on the vector ALU underneath
//   B0  dV, dK from rows 0-31, with P and dS of rows 32-63 underneath                  B1  dV, dK from rows 32-63
// and the LDS operand of instruction i + BWD_RING is requested right after instruction i is issued.  The S and dP
// accumulators do not start from zero but from -L_i log2(e) and -D_i (staged per tile next to the Q and dO rows), so
// P = exp2(S) and dS = P * dP need no subtraction.
template <typename T>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void sdpa_bwd_dkv_kernel(SdpaBwdParams bp)
{
#if defined(__HIP_DEVICE_COMPILE__)
    typedef typename Mma<T>::vec8 vec8;
    typedef PfLayout<128> L;
    typedef float float4v __attribute__((ext_vector_type(4)));
    constexpr int NSTEP = 8, NDB = 4, R = BWD_RING;
    constexpr int STAGE = 2 * L::TILE_BYTES + 1024;     // Q rows, dO rows, 64 x -L_i log2(e), 64 x -D_i (and padding)
    const SdpaParams& p = bp.f;
    __shared__ __attribute__((aligned(1024))) char smem[2 * STAGE];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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
    const int my_j = j0 + wave * 32 + ql;              // this lane's key

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
    const int i_all_wave = p.causal ? max(j0 + wave * 32 + 31 - coff, 0) : 0;
    const int t_begin = i_begin_wg / PF_BN;
    const int n_qt = (Sq + PF_BN - 1) / PF_BN;
    const int tiles_per_head = j0 < kv_len ? max(n_qt - t_begin, 0) : 0;
    const int n_tiles = tiles_per_head * p.G;           // the group's query heads one after another

    BwdTiles<T> tl;
    tl.init(wave, lane, p.q_ss, bp.do_ss);

    // this lane's key: K row (scaled into log2 units) and V row as B operands
    vec8 kreg[NSTEP], vreg[NSTEP];
    {
        const int kj = min(my_j, Skv - 1);
        const T* krow = kp + (int64_t)kj * p.k_ss + g * 8;
        const T* vrow = vp + (int64_t)kj * p.v_ss + g * 8;
        const float c2 = p.scale * 1.4426950408889634f;
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
            vec8 x = *(const vec8*)(krow + s * 16);
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = (T)((float)x[e] * c2);
            kreg[s] = x;
            vreg[s] = *(const vec8*)(vrow + s * 16);
        }
    }
    // rows i >= lo_i see this lane's key under the causal mask
    const int lo_i = p.causal ? my_j - coff : -0x40000000;

    floatx16 dk_acc[NDB], dv_acc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) { dk_acc[db][r] = 0.0f; dv_acc[db][r] = 0.0f; }

    // The copies walk the tiles with running addresses (the wavefront issues one instruction every four clocks and has
    // the SIMD to itself: index arithmetic per tile would cost as much as the matrix instructions it feeds).
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
        nx_rows = Sq - r0;
        nx_qrem = (int64_t)(nx_rows - 1) * p.q_ss * 2 + 256;
        nx_grem = (int64_t)(nx_rows - 1) * bp.do_ss * 2 + 256;
        nx_r = 0;
        nx_h = h;
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

    auto tile = [&](int stage, int i0) __attribute__((always_inline)) {
        const char* qt = smem + stage * STAGE;
        const char* gt = qt + L::TILE_BYTES;
        const char* nl = gt + L::TILE_BYTES;
        // matrix instruction i of the tile: its LDS operand ...
        vec8 ring[R];
        auto fetch = [&](int i) __attribute__((always_inline)) {
            if (i < 32) {
                const int qb = i / 16, s = (i % 16) / 2, which = i % 2;
                ring[i % R] = tl.rows_op(which ? gt : qt, qb, s);
            } else {
                const int j = i - 32, qb = j / 16, h = (j % 16) / 8, db = (j % 8) / 2, which = 1 - j % 2;
                ring[i % R] = tl.tr_op(which ? gt : qt, db, 2 * qb + h);
            }
        };
        floatx16 sa[2], da[2];
        vec8 pp[2][2], ds[2][2];
        // ... and the instruction itself
        auto mma = [&](int i) __attribute__((always_inline)) {
            if (i < 32) {
                const int qb = i / 16, s = (i % 16) / 2;
                if (i % 2 == 0) sa[qb] = Mma<T>::run(ring[i % R], kreg[s], sa[qb]);
                else da[qb] = Mma<T>::run(ring[i % R], vreg[s], da[qb]);
            } else {
                const int j = i - 32, qb = j / 16, h = (j % 16) / 8, db = (j % 8) / 2;
                if (j % 2 == 0) dv_acc[db] = Mma<T>::run(ring[i % R], pp[qb][h], dv_acc[db]);
                else dk_acc[db] = Mma<T>::run(ring[i % R], ds[qb][h], dk_acc[db]);
            }
        };
        // S and dP of a query block leave the accumulation registers in one go, at the seam between two runs, where the
        // matrix pipe drains anyway: a read of an accumulation register waits until no matrix instruction is in
        // flight (about one instruction's time each when the reads are spread among them).
        float sv[16], dv[16];
        auto take = [&](int qb) __attribute__((always_inline)) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                sv[r] = sa[qb][r];
                dv[r] = da[qb][r];
                asm volatile("" : "+v"(sv[r]), "+v"(dv[r]));
            }
        };
        // P and dS of register r of query block qb (row i0 + 32*qb + 8*(r/4) + 4*g + (r%4)), rounded for the next products
        auto soft = [&](int qb, int r) __attribute__((always_inline)) {
            const float pr = __builtin_amdgcn_exp2f(sv[r]);
            pp[qb][r / 8][r % 8] = (T)pr;
            ds[qb][r / 8][r % 8] = (T)(pr * dv[r]);
        };

        // The accumulators start from -L_i log2(e) and -D_i.  What the mask hides starts from -inf instead and ends as
        // P = 0, dS = 0 * (finite): only the causal edge needs that here, rows past Sq arrive as zeros throughout (dO = 0,
        // dP = 0), rows without any visible key carry -inf already, and keys past kv_len are zeroed at the end.
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const float4v a = *(const float4v*)(nl + (32 * qb + 8 * r4 + 4 * g) * 4);
                const float4v d = *(const float4v*)(nl + 256 + (32 * qb + 8 * r4 + 4 * g) * 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) { sa[qb][4 * r4 + e] = a[e]; da[qb][4 * r4 + e] = d[e]; }
            }
#pragma unroll
        for (int i = 0; i < R; ++i) fetch(i);
        if (i0 < i_all_wave) {          // some row of the tile does not see every key of this wavefront
            const int rel = lo_i - i0 - 4 * g;
#pragma unroll
            for (int qb = 0; qb < 2; ++qb)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (32 * qb + 8 * (r / 4) + (r % 4) < rel) sa[qb][r] = -INFINITY;
        }
        __builtin_amdgcn_sched_barrier(0);
        // The order is pinned two matrix instructions at a time (the scheduler, left a whole run, strings the
        // instructions of one accumulator together, each waiting for the one before).
#pragma unroll
        for (int i = 0; i < 16; i += 2) {       // A0
            mma(i); mma(i + 1);
            fetch(i + R); fetch(i + R + 1);
            __builtin_amdgcn_sched_barrier(0);
        }
        take(0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 16; i < 32; i += 2) {      // A1 over the vector work of rows 0-31
            mma(i); mma(i + 1);
            fetch(i + R); fetch(i + R + 1);
            soft(0, i - 16); soft(0, i - 15);
            __builtin_amdgcn_sched_barrier(0);
        }
        take(1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 32; i < 48; i += 2) {      // B0 over the vector work of rows 32-63
            mma(i); mma(i + 1);
            fetch(i + R); fetch(i + R + 1);
            soft(1, i - 32); soft(1, i - 31);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int i = 48; i < 64; i += 2) {      // B1
            mma(i); mma(i + 1);
            if (i + R < 64) { fetch(i + R); fetch(i + R + 1); }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    if (n_tiles > 0) {
        to_head(0);
        issue(0);
    }
    int i0 = t_begin * PF_BN;
    for (int t = 0; t < n_tiles; ++t) {
        // tile t has landed for everyone and everyone is done with tile t-1: the other stage is free
        __builtin_amdgcn_s_waitcnt(0x0F70);             // vmcnt(0)
        asm volatile("" ::: "memory");
        __syncthreads();
        if (t + 1 < n_tiles) issue((t + 1) & 1);
        // (The K and V rows are pinned to the architectural half of the register file: the accumulators - dK, dV and
        // the tile's S and dP, 192 registers - then fit the accumulation half together, where dK and dV are pinned in
        // turn.  Left alone, the register allocator parks dK and dV in the architectural half around every tile.)
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) asm volatile("" : "+v"(kreg[s]), "+v"(vreg[s]));
#pragma unroll
        for (int db = 0; db < NDB; ++db) asm volatile("" : "+a"(dk_acc[db]), "+a"(dv_acc[db]));
        // Every wavefront computes every tile: one whose keys no row of the tile sees (the first tile or two under a
        // causal mask) works on -inf, and would wait at the next barrier for the others anyway.  A tile skipped by
        // some is also a second path the accumulators take around the loop, which costs register shuffling.
        tile(t & 1, i0);
        i0 += PF_BN;
        if (i0 >= n_qt * PF_BN) i0 = t_begin * PF_BN;       // next head of the group
    }

    if (my_j < Skv) {
        T* krow = dkp + (int64_t)my_j * bp.dk_ss;
        T* vrow = dvp + (int64_t)my_j * bp.dv_ss;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                typedef T vec4 __attribute__((ext_vector_type(4)));
                vec4 wk, wv;
#pragma unroll
                for (int e = 0; e < 4; ++e) {       // (a key past kv_len met no mask above: its sums are not gradients)
                    wk[e] = (T)(my_j < kv_len ? dk_acc[db][r4 * 4 + e] * p.scale : 0.0f);
                    wv[e] = (T)(my_j < kv_len ? dv_acc[db][r4 * 4 + e] : 0.0f);
                }
                *(vec4*)(krow + db * 32 + r4 * 8 + g * 4) = wk;
                *(vec4*)(vrow + db * 32 + r4 * 8 + g * 4) = wv;
            }
    }
#endif
}

template <typename T>
static hipError_t launch_bwd_t(const SdpaBwdParams& bp, hipStream_t stream)
{
    const SdpaParams& p = bp.f;
    const int64_t rows = (int64_t)p.B * p.Hq * p.Sq;
    if (rows > 0) {
        hipLaunchKernelGGL((sdpa_bwd_delta_kernel<T>), dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, stream, bp);
        const int nqb = (p.Sq + PF_BM - 1) / PF_BM;
        const int64_t total = (int64_t)nqb * p.Hq * p.B;
        SdpaBwdParams bq = bp;      // two workgroups per CU, an eighth of the CUs per XCD
        bq.f.interleave = work_interleave(p.causal != 0, 2 * device_cus() / 8, p.G, nqb, (total & 7) == 0 ? total >> 3 : total);
        bq.f.deal_groups = (total & 7) == 0 ? work_deal(bq.f.interleave, p.G, nqb, total >> 3) : 0;
        hipLaunchKernelGGL((sdpa_bwd_dq_kernel<T>), dim3((unsigned)total), dim3(256), 0, stream, bq);
    }
    const int nkb = (p.Skv + BWD_KEYS - 1) / BWD_KEYS;
    if ((int64_t)nkb * p.Hkv * p.B > 0)
        hipLaunchKernelGGL((sdpa_bwd_dkv_kernel<T>), dim3((unsigned)((int64_t)nkb * p.Hkv * p.B)), dim3(256), 0, stream, bp);
    return hipGetLastError();
}

// Host has validated: dtype f16/bf16, D == Dv == 128, no dense mask, unit last-axis strides, 16-byte aligned rows,
// row strides below 2^24 elements, lse and the delta workspace present.
hipError_t launch_sdpa_bwd_mfma(const SdpaBwdParams& bp, int dtype, hipStream_t stream)
{
    if (dtype == 1) return launch_bwd_t<f16_t>(bp, stream);
    return launch_bwd_t<bf16_t>(bp, stream);
}

}  // namespace incin_rocm
