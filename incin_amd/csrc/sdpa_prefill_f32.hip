// f32 attention forward on the gfx950 matrix cores with IEEE single-precision arithmetic
// (v_mfma_f32_32x32x2_f32: f32 operands, f32 products and sums - no reduced-precision path), for head dimensions up to
// 128 (instances for 64 and 128; a smaller D or Dv, in whole 16-byte vectors, is zero-padded on the way into LDS), optional causal mask, per-batch key lengths, a dense additive mask with arbitrary broadcast strides,
// MHA and GQA.  f32 is the one dtype the reference's own operator runs end to end
// (crates/incin-backends/src/cpu/ops/shape_ops.rs:1245-1269 over cpu/ops/matmul.rs:234,254), with a 1e-5 bar.
//
// Shape of the computation - that of sdpa_prefill_mfma.hip (one workgroup = 4 wavefronts = 128 query rows, one
// wavefront = 32 query rows), with the operand layouts of the k = 2 instruction:
//
//   S^T = K_blk Q'^T   A = K: lane (key = lane % 32, g = lane / 32) supplies K[key][d]; B = Q'^T: the same lane
//                      supplies Q'[query = lane % 32][d] (Q' = Q * scale * log2(e), kept in registers for the whole
//                      kernel).  One instruction sums over two values of d: the one the g = 0 lanes hold and the one
//                      the g = 1 lanes hold.  Which two is free as long as A and B agree, so a lane reads four
//                      consecutive floats d = 8j + 4g .. 8j + 4g + 3 (one 16-byte LDS read) and they serve four
//                      instructions.  In the 32 x 32 result a lane owns ONE query (column lane % 32) and 16 keys
//                      (register r is key 8 (r / 4) + 4 g + r % 4): row maximum and row sum are in-lane reductions
//                      plus one exchange with lane ^ 32.
//   P^T                exp2 of that in registers; the accumulator layout of S^T is already the B-operand layout of
//                      the next product: register r is the k-step of keys kappa(r, 0), kappa(r, 1).
//   O^T += V^T P^T     A = V^T: lane (d = lane % 32, g) supplies V[kappa(r, g)][32 db + d]: a 4-byte LDS read of
//                      32 consecutive floats of one row per half-wavefront; no transposition anywhere.
//
// A dense additive mask comes with one flag per block of 32 rows x 32 keys (mask_blocks.hip): blocks the mask hides
// completely are skipped, blocks where it is zero run without it, the rest add its values to the scores.
//
// The matrix pipe is the bound by a wide margin (an instruction occupies it for 64 cycles and needs one register of
// each operand), so the loop is plain: per key tile one barrier, the global -> LDS copies of the next tile (K and V,
// two buffers each, 16 KiB tiles: 64 keys at D = 64, 32 at D = 128), scores, exact online softmax, second product.
// The other wavefront of the SIMD covers the vector work.  LDS rows are unpadded with their 16-byte chunks
// XOR-swizzled by the row number so that both read patterns touch every bank once.
#include <type_traits>

#include "sdpa_mfma_common.h"

namespace incin_rocm {

// SPLIT: the launch is a grid of (work items) x (splits of the key axis); a workgroup handles the keys of its split only and
// writes, per row, the unnormalised O, the maximum and the sum in the partial-result format of the split-KV kernels, whose
// combine kernel finishes - for launches with too few (batch, head, row block) items to fill the device over a long key axis.
template <int D, bool DENSE, bool SPLIT = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void sdpa_prefill_f32_kernel(SdpaParams p)
{
#if defined(__HIP_DEVICE_COMPILE__)   // the body uses device-only types (buffer descriptors); the host pass needs only the stub
    typedef F32Layout<D> L;
    typedef float float4v __attribute__((ext_vector_type(4)));
    constexpr int NJ = D / 8;              // groups of four k-steps of the S^T product
    constexpr int NDB = D / 32;            // 32-wide blocks of the head dimension
    constexpr int LPW = L::LOADS_PER_WAVE;
    constexpr int KT = L::KT, NB = L::NB;

    __shared__ __attribute__((aligned(1024))) char smem[4 * L::TILE_BYTES];   // K buffers 0, 1, V buffers 0, 1

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ql = lane & 31, g = lane >> 5;
    const int Sq = p.Sq, Skv = p.Skv;

    // ---- which (batch, head, query block): the work order of the 16-bit kernels (longest blocks first, an XCD keeps
    // the heads that share K/V) -----------------------------------------------------------------------------------
    const int nqb = (Sq + PF_BM - 1) / PF_BM;
    const int total = gridDim.x;
    const WorkItem wi = (total & 7) == 0 ? work_item_of_share(blockIdx.x & 7, blockIdx.x >> 3, total >> 3, p.interleave, p.G, nqb, p.deal_groups)
                                         : work_item(blockIdx.x, p.interleave, p.G, nqb);
    const int gq = wi.gq, qb = wi.qblk, bhkv = wi.bhkv;
    const int hkv = bhkv % p.Hkv, b = bhkv / p.Hkv;
    const int hq = hkv * p.G + gq;
    const int q0 = qb * PF_BM;

    const float* qp = (const float*)p.q + (int64_t)b * p.q_sb + (int64_t)hq * p.q_sh;
    const float* kp = (const float*)p.k + (int64_t)b * p.k_sb + (int64_t)hkv * p.k_sh;
    const float* vp = (const float*)p.v + (int64_t)b * p.v_sb + (int64_t)hkv * p.v_sh;
    float* op = (float*)p.o + (int64_t)b * p.o_sb + (int64_t)hq * p.o_sh;

    int kv_len = Skv;
    if (p.kv_lens) kv_len = clampi(p.kv_lens[b], 0, Skv);
    // a split ends where the next begins: to this workgroup the keys beyond do not exist (split_len is a multiple of the tile)
    const int split = SPLIT ? (int)blockIdx.y : 0;
    if (SPLIT) kv_len = min(kv_len, (split + 1) * p.split_len);
    const int rows_b = p.q_lens ? clampi(p.q_lens[b], 0, Sq) : Sq;      // query rows at and beyond are padding
    if (q0 >= rows_b) return;                                           // (uniform: before any barrier)
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
    if (q0 + wave * 32 >= rows_b) lim_wave_min = lim_wave_max = 0;      // a wavefront of padding rows only keeps the barriers company
    if (DENSE && p.mask_lims != nullptr) {
        // a launch of the f32 split-KV kernel went before this one and computed the 128-row blocks whose mask rows are all n
        // zeros and then -inf from their limits (sdpa_decode_f32.hip, LIMS): such a block is done
        __shared__ int s_ok[4];
        const bool no_limit = my_i < rows_b && mask_lims_of(p, b, hq)[p.m_si ? my_i : 0] < 0;
        const bool wave_ok = __builtin_amdgcn_ballot_w64(no_limit) == 0;
        if (lane == 0) s_ok[wave] = wave_ok ? 1 : 0;
        __syncthreads();
        if ((s_ok[0] & s_ok[1] & s_ok[2] & s_ok[3]) != 0) return;      // (uniform)
    }
    const int n_tiles = (j_end + KT - 1) / KT;
    const int t_first = SPLIT ? min(split * (p.split_len / KT), n_tiles) : 0;
    const int n_act = lim_wave_max > 0 ? (lim_wave_max + KT - 1) / KT : 0;      // tiles this wavefront computes

    // ---- global -> LDS copy plan: wavefront-wide load ii = wave * LPW + c fills LDS bytes [ii * 1024, +1024) of a tile
    int k_voff[LPW], v_voff[LPW];
#pragma unroll
    for (int c = 0; c < LPW; ++c) {
        const int pos = (wave * LPW + c) * 64 + lane;
        const int row = pos / L::CPR, slot = pos % L::CPR;
        k_voff[c] = dma_chunk_offset(row, (int)p.k_ss * 4, slot ^ L::f(row), p.D * 4);
        v_voff[c] = dma_chunk_offset(row, (int)p.v_ss * 4, slot ^ L::f(row), p.Dv * 4);
    }
    const int64_t k_tile_bytes = (int64_t)KT * p.k_ss * 4, v_tile_bytes = (int64_t)KT * p.v_ss * 4;
    auto issue = [&](const float* base, int64_t tile_bytes, int64_t row_stride, int row_floats, int t, int buf, const int (&voff)[LPW]) __attribute__((always_inline)) {
        // bytes to the end of the last row this workgroup may see: loads past that return 0 (rows past a batch
        // entry's key count are never read)
        int64_t rem = (int64_t)(j_end - t * KT - 1) * row_stride * 4 + row_floats * 4;
        if (rem > 0x7fffffffLL) rem = 0x7fffffffLL;
        const uint4v r = dma_descriptor((const char*)base + t * tile_bytes, (int)rem);
        const unsigned dst = lds_address(smem) + buf * L::TILE_BYTES + wave * LPW * 1024;
#pragma unroll
        for (int c = 0; c < LPW; ++c) dma_copy16(r, dst + c * 1024, voff[c]);
    };
    auto issue_kv = [&](int t) __attribute__((always_inline)) {
        issue(kp, k_tile_bytes, p.k_ss, p.D, t, t & 1, k_voff);
        issue(vp, v_tile_bytes, p.v_ss, p.Dv, t, 2 + (t & 1), v_voff);
    };

    // ---- LDS read addresses (bytes inside a tile buffer), kept to a few registers: the rest is one vector
    // instruction per read, which costs nothing beside a 64-cycle matrix instruction ---------------------------------
    // K operand: lane (ql, g) reads row 32 kb + ql, logical chunk 2 j + g, stored at chunk (2 j + g) ^ f(ql).  With
    // f = f_hi | f_0 (bit 0 apart): byte address = [ql * ROWB + ((g ^ f_0) << 4) + (f_hi << 4)] ^ (j << 5); the
    // three terms in brackets share no bits, and neither does j << 5 with the first two.
    const int k_base = ql * L::ROWB + (((g ^ L::f(ql)) & 1) << 4) + ((L::f(ql) & 0xe) << 4);
    auto k_addr = [&](int j) __attribute__((always_inline)) { return k_base ^ (j << 5); };
    // V operand of k-step r, block db: row 8 (r / 4) + 4 g + r % 4 of the 32-key block, float 32 db + ql, i.e. logical
    // chunk 8 db + ql / 4 at chunk slot (8 db + ql / 4) ^ f(row), f(row) = r % 4 | 4 (r / 4 % 2) | 8 g: the low three
    // bits of the slot are (ql / 4) ^ c with c = r % 4 | 4 (r / 4 % 2), the rest is db ^ g.
    int v_low[8], v_high[NDB];
#pragma unroll
    for (int c = 0; c < 8; ++c) v_low[c] = 4 * g * L::ROWB + (((ql >> 2) ^ c) << 4) + (ql & 3) * 4;
#pragma unroll
    for (int db = 0; db < NDB; ++db) v_high[db] = (db ^ g) << 7;

    // ---- Q'^T operand, resident in registers ----------------------------------------------------------------------
    // (fetched 16 bytes per lane, eight lanes to a 128-byte run of a row, and brought into the operand layout through this
    // wavefront's 4 KiB of the K buffer the first copies do not fill: nothing is copied there before the loop's first barrier)
    float4v qreg[NJ];
    {
        uint4v qraw[NJ / 4][4];
        fetch_q_rows(qraw, qp, q0 + wave * 32, Sq, p.q_ss, p.D, lane);
        stage_q_rows(qreg, qraw, smem + ((t_first + 1) & 1) * L::TILE_BYTES + wave * 4096, lane);
        const float c2 = p.scale * 1.4426950408889634f;      // scores in log2 units
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) qreg[j][e] *= c2;
    }
    const float* mrow = nullptr;          // this lane's row of the dense mask
    const uint8_t* mflags = nullptr;      // block flags of this wavefront's 32 rows: 0 mixed, 1 all zero, 2 all -inf
    if (DENSE) {
        mrow = (const float*)p.mask + (int64_t)b * p.m_sb + (int64_t)hq * p.m_sh + (int64_t)min(my_i, Sq - 1) * p.m_si;
        mflags = mask_flags_of(p, b, hq) + (int64_t)((q0 >> 5) + wave) * ((Skv + 31) / 32);
    }

    floatx16 o_acc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[db][r] = 0.0f;
    float m_run = -INFINITY;      // running maximum (log2 units) of this lane's query, the same in lanes l and l ^ 32
    float l_run = 0.0f;           // this lane's share of the running denominator

    if (n_tiles > t_first) issue_kv(t_first);
    for (int t = t_first; t < n_tiles; ++t) {
        // K(t), V(t) have arrived for everyone, everyone is done with tile t - 1: its buffers take tile t + 1
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (t + 1 < n_tiles) issue_kv(t + 1);
        if (t >= n_act) continue;
        const char* kb_ = smem + (t & 1) * L::TILE_BYTES;
        const char* vb_ = smem + (2 + (t & 1)) * L::TILE_BYTES;
#pragma unroll
        for (int kb = 0; kb < NB; ++kb) {
            const int j0 = t * KT + kb * 32;
            if (j0 >= lim_wave_max) break;                    // (uniform) nothing of this block is visible to the wavefront
            int flag = 1;
            if (DENSE) {
                flag = __builtin_amdgcn_readfirstlane((int)mflags[j0 >> 5]);
                if (flag == 2) continue;                      // the mask hides the whole block from these rows
            }
            // dense mask values of this lane's 16 keys, fetched ahead of the product that hides their latency
            float mv[16];
            if (DENSE && flag == 0) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int j = min(j0 + 8 * (r / 4) + 4 * g + (r % 4), Skv - 1);
                    mv[r] = mrow[(int64_t)j * p.m_sj];
                }
            }
            // ---- scores: two chains over the halves of the head dimension -------------------------------------
            floatx16 s0, s1;
#pragma unroll
            for (int r = 0; r < 16; ++r) { s0[r] = 0.0f; s1[r] = 0.0f; }
#pragma unroll
            for (int j = 0; j < NJ / 2; ++j) {
                const float4v ka = *(const float4v*)(kb_ + kb * 32 * L::ROWB + k_addr(j));
                const float4v kc = *(const float4v*)(kb_ + kb * 32 * L::ROWB + k_addr(j + NJ / 2));
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[e], qreg[j][e], s0, 0, 0, 0);
                    s1 = __builtin_amdgcn_mfma_f32_32x32x2f32(kc[e], qreg[j + NJ / 2][e], s1, 0, 0, 0);
                }
            }
            floatx16 s;
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] = s0[r] + s1[r];
            if (DENSE && flag == 0) {
#pragma unroll
                for (int r = 0; r < 16; ++r) s[r] = __builtin_fmaf(mv[r], 1.4426950408889634f, s[r]);
            }
            if (j0 + 32 > lim_wave_min) {                     // (uniform) the block crosses a limit of this wavefront
                const int rel = lim_lane - (j0 + 4 * g);
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (8 * (r / 4) + (r % 4) >= rel) s[r] = -INFINITY;
            }
            // ---- online softmax ------------------------------------------------------------------------------------
            float tmax = s[0];
#pragma unroll
            for (int r = 1; r < 16; ++r) tmax = fmaxf(tmax, s[r]);
            tmax = xor32_max(tmax);
            const float m_new = fmaxf(m_run, tmax);
            const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);       // exp2(-inf) = 0: nothing accumulated yet
            m_run = m_new;
            float rsum = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                s[r] = __builtin_amdgcn_exp2f(s[r] - m_use);
                rsum += s[r];
            }
            l_run = l_run * alpha + rsum;
            if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
                for (int db = 0; db < NDB; ++db)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o_acc[db][r] *= alpha;
            }
            // ---- O^T += V^T P^T: k-step r takes keys kappa(r, 0), kappa(r, 1) ------------------------------------
            const char* vblk = vb_ + kb * 32 * L::ROWB;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float vv[NDB];
#pragma unroll
                for (int db = 0; db < NDB; ++db)
                    vv[db] = *(const float*)(vblk + ((r / 8) * 16 + 8 * ((r / 4) % 2) + r % 4) * L::ROWB + v_low[(r % 4) | (4 * ((r / 4) % 2))] + v_high[db]);
#pragma unroll
                for (int db = 0; db < NDB; ++db) o_acc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv[db], s[r], o_acc[db], 0, 0, 0);
            }
        }
    }

    // ---- normalise and store --------------------------------------------------------------------------------------
    const float l_tot = xor32_sum(l_run);
    if constexpr (SPLIT) {
        // partial result of this split: unnormalised O, and (maximum, sum) in the natural-log units the combine kernel takes
        // for f32 storage; a row that saw no key in this split has the maximum -inf
        if (my_i < rows_b) {
            const int64_t slot = (((int64_t)b * p.Hq + hq) * Sq + my_i) * p.num_splits + split;
            float* arow = p.ws_acc + slot * D + g * 4;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    float4v w = {o_acc[db][r4 * 4], o_acc[db][r4 * 4 + 1], o_acc[db][r4 * 4 + 2], o_acc[db][r4 * 4 + 3]};
                    *(float4v*)(arow + db * 32 + r4 * 8) = w;
                }
            if (g == 0) {
                p.ws_ml[slot * 2 + 0] = l_tot == 0.0f ? -INFINITY : m_run * 0.6931471805599453f;
                p.ws_ml[slot * 2 + 1] = l_tot;
            }
        }
        return;
    }
    const float inv = (l_tot == 0.0f) ? __builtin_nanf("") : 1.0f / l_tot;   // no visible key: NaN, as the reference
    if (p.lse && g == 0 && my_i < rows_b)
        p.lse[((int64_t)b * p.Hq + hq) * Sq + my_i] = l_tot == 0.0f ? -INFINITY : (m_run + __builtin_log2f(l_tot)) * 0.6931471805599453f;
    // through this wavefront's 4 KiB of the K buffer the last tile did not use (every wavefront is past the barrier of that
    // tile, i.e. done with the tile before it, and nothing has been copied since)
    store_o_rows_f32(o_acc, inv, smem + (n_tiles & 1) * L::TILE_BYTES + wave * 4096, op, q0 + wave * 32, rows_b, p.o_ss, p.Dv, lane);
#endif
}

hipError_t launch_sdpa_combine(const SdpaParams& p, int dtype, hipStream_t stream);

template <int D, bool DENSE>
static hipError_t launch_prefill_f32_t(const SdpaParams& p0, hipStream_t stream)
{
    SdpaParams p = p0;
    const int nqb = (p.Sq + PF_BM - 1) / PF_BM;
    const int64_t total = (int64_t)nqb * p.Hq * p.B;
    if (total <= 0) return hipSuccess;
    if (total > 0x7fffffffLL) return hipErrorInvalidValue;
    p.interleave = work_interleave(p.causal != 0 || p.mask != nullptr, 2 * device_cus() / 8, p.G, nqb, (total & 7) == 0 ? total >> 3 : total);
    p.deal_groups = (total & 7) == 0 ? work_deal(p.interleave, p.G, nqb, total >> 3, p.causal != 0 || p.mask != nullptr) : 0;
    if constexpr (!DENSE) {
        if (p.num_splits > 1) {          // split launch: partial results, then the split-KV kernels' combine pass
            hipLaunchKernelGGL((sdpa_prefill_f32_kernel<D, false, true>), dim3((unsigned)total, (unsigned)p.num_splits), dim3(256), 0, stream, p);
            hipError_t e = hipGetLastError();
            return e != hipSuccess ? e : launch_sdpa_combine(p, 0, stream);
        }
    }
    hipLaunchKernelGGL((sdpa_prefill_f32_kernel<D, DENSE>), dim3((unsigned)total), dim3(256), 0, stream, p);
    return hipGetLastError();
}

// Host has validated: f32, D and Dv <= 128 in whole 16-byte vectors (p.Dp = the instance: 64 or 128), finite scale, rows 16-byte aligned with unit last-dim stride, row
// strides below 2^24 elements (tile offsets fit the 32-bit buffer offset); the dense mask, if any, has any strides.
hipError_t launch_sdpa_prefill_f32(const SdpaParams& p, hipStream_t stream)
{
    if (p.mask) return p.Dp == 128 ? launch_prefill_f32_t<128, true>(p, stream) : launch_prefill_f32_t<64, true>(p, stream);
    return p.Dp == 128 ? launch_prefill_f32_t<128, false>(p, stream) : launch_prefill_f32_t<64, false>(p, stream);
}

}  // namespace incin_rocm
