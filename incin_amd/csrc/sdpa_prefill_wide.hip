// bf16 / f16 attention forward on the gfx950 matrix cores for head dimensions above 128 (up to 256, D and Dv in whole
// 16-byte vectors, zero-padded into the 256 instance on the way into LDS) on prefill shapes: the function of the
// reference CPU composition (crates/incin-backends/src/cpu/ops/shape_ops.rs:1245-1269), optional causal mask, per-batch
// key and query lengths, MHA and GQA.
//
// Decode shapes at these head dimensions run on the split-KV kernel's 256 instance (sdpa_decode_mfma.hip), and so did
// prefill shapes before this kernel: 32 rows per workgroup there, each workgroup streaming K and V for itself, which
// makes the traffic between L2 and LDS the bound (340 - 460 TFLOP/s).  Here a workgroup is 4 wavefronts = 128 query
// rows sharing every K / V tile, the shape of sdpa_prefill_mfma.hip with the operand layouts of sdpa_decode_mfma.hip:
//
//   S^T = K_tile Q^T     v_mfma_f32_32x32x16 over the 16 k-steps of 256 elements: A = K rows from LDS (16-byte reads),
//                        B = Q^T resident in registers (64 of them); a lane owns one query and 16 keys of the tile.
//   softmax              scale * log2(e) folded into Q (any finite scale), masks as -inf before the maximum, the
//                        reference maximum moved lazily (threshold 2^8), P rounded to the storage type in registers.
//   O^T += V^T P^T       A = V^T through the transposing LDS read, 8 blocks of 32 columns: 128 accumulator registers.
//
// A tile is 32 keys (16 KiB of K, 16 KiB of V), two buffers each: 64 KiB of LDS and 256 registers per lane, so two
// workgroups share a compute unit and one's softmax runs beside the other's matrix instructions.  One barrier per tile:
// it publishes tile t, whose copies (global -> LDS, no register staging) were started an iteration earlier, and frees
// the buffers of tile t - 1 for the copies of tile t + 1.  The loop is the plain one - with two matrix instructions per
// key and row where head dimension 128 has one, the vector work between them weighs half as much.
#include "sdpa_mfma_common.h"

namespace incin_rocm {

constexpr int PW_KT = 32;      // keys per tile

// DENSE: a dense additive mask (any broadcast strides) comes with one flag per block of 32 rows x 32 keys (mask_blocks.hip) -
// a tile of this kernel is one such block per wavefront: tiles where the mask is zero run without it, the others add its
// values to the scores, and the tiles before the first and after the last one it shows to a wavefront are skipped.
//
// SPLIT: a grid of (work items) x (splits of the key axis), as in sdpa_prefill_mfma.hip - a workgroup handles the keys of its
// split and writes, per row, the unnormalised O, the reference and the sum in the split-KV kernels' partial-result format; their
// combine kernel finishes.  For launches with few 128-row blocks over a long key axis (a chunk of a long prompt).
//
// MASK: 0 no mask tensor; 1 (DENSE) a dense additive mask by flags and values; 2 (LIMS) the launch for the 128-row blocks all
// of whose rows the mask gives n zeros and then -inf (sdpa_prefill_mfma.hip has the scheme: a masked request is the LIMS
// launch, whose other workgroups leave at once, and then the DENSE launch, whose workgroups leave if LIMS took their block).
template <typename T, int MASK, bool SPLIT = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void sdpa_prefill_wide_kernel(SdpaParams p)
{
    constexpr bool DENSE = MASK == 1, LIMS = MASK == 2;
#if defined(__HIP_DEVICE_COMPILE__)
    typedef typename Mma<T>::vec8 vec8;
    constexpr int D = 256;
    typedef PfLayout<D> L;
    constexpr int NSTEP = D / 16, NDB = D / 32;
    constexpr int TILE = PW_KT * L::ROWB;              // 16 KiB
    constexpr int LPW = TILE / 1024 / 4;               // wavefront-wide 1 KiB copies per tensor per tile: 4
    __shared__ __attribute__((aligned(1024))) char smem[4 * TILE];      // K buffers 0, 1, V buffers 0, 1

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ql = lane & 31, g = lane >> 5;
    const int Sq = p.Sq, Skv = p.Skv;

    // ---- which (batch, head, query block): the work order of the other prefill kernels ---------------------------------
    const int nqb = (Sq + PF_BM - 1) / PF_BM;
    const int total = gridDim.x;
    const WorkItem wi = (total & 7) == 0 ? work_item_of_share(blockIdx.x & 7, blockIdx.x >> 3, total >> 3, p.interleave, p.G, nqb, p.deal_groups)
                                         : work_item(blockIdx.x, p.interleave, p.G, nqb);
    const int hkv = wi.bhkv % p.Hkv, b = wi.bhkv / p.Hkv;
    const int hq = hkv * p.G + wi.gq;
    const int q0 = wi.qblk * PF_BM;

    const T* qp = (const T*)p.q + (int64_t)b * p.q_sb + (int64_t)hq * p.q_sh;
    const T* kp = (const T*)p.k + (int64_t)b * p.k_sb + (int64_t)hkv * p.k_sh;
    const T* vp = (const T*)p.v + (int64_t)b * p.v_sb + (int64_t)hkv * p.v_sh;
    T* op = (T*)p.o + (int64_t)b * p.o_sb + (int64_t)hq * p.o_sh;

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
    int n_tiles = (j_end + PW_KT - 1) / PW_KT;
    int n_act = lim_wave_max > 0 ? (lim_wave_max + PW_KT - 1) / PW_KT : 0;      // tiles this wavefront computes: [w_first, n_act)
    int w_first = 0, t_first = SPLIT ? min(split * (p.split_len / PW_KT), n_tiles) : 0;
    // dense mask: this lane's row of it and the flags of this wavefront's 32 rows, one per tile.  The tiles before the first
    // and after the last one the mask shows to a wavefront are not computed (a sliding window's past), and the workgroup's
    // copies run from the first to the last tile any of its wavefronts computes; a hidden tile in between goes through the
    // mask's values like a mixed one (-inf everywhere).
    const T* mrow = nullptr;
    const uint8_t* mflags = nullptr;
    __shared__ int s_range[8];
    if ((DENSE || LIMS) && p.mask_lims != nullptr) {
        // does every row of this workgroup have a limit?  One exchange through LDS says that and, for LIMS, the largest limit.
        const int32_t* lims = mask_lims_of(p, b, hq);
        const bool row_here = my_i < rows_b;
        const int lm = lims[p.m_si ? min(my_i, Sq - 1) : 0];
        const bool wave_ok = __builtin_amdgcn_ballot_w64(row_here && lm < 0) == 0;
        if (LIMS) {
            // this lane's limit, the smallest and largest of the wavefront
            lim_lane = row_here ? min(lim_lane, lm) : 0;
            int lo = row_here ? lim_lane : 0x7fffffff, hi = lim_lane;
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) {
                lo = min(lo, __shfl_xor(lo, off, 64));
                hi = max(hi, __shfl_xor(hi, off, 64));
            }
            lim_wave_min = __builtin_amdgcn_readfirstlane(lo == 0x7fffffff ? 0 : lo);
            lim_wave_max = __builtin_amdgcn_readfirstlane(hi);
        }
        if (lane == 0) { s_range[wave] = wave_ok ? 1 : 0; s_range[4 + wave] = lim_wave_max; }
        __syncthreads();
        const bool all = __builtin_amdgcn_readfirstlane((s_range[0] & s_range[1] & s_range[2] & s_range[3]) != 0 ? 1 : 0) != 0;
        if (all != LIMS) return;                           // the other launch computes this block
        if (LIMS) {
            j_end = __builtin_amdgcn_readfirstlane(max(max(s_range[4], s_range[5]), max(s_range[6], s_range[7])));
            n_tiles = (j_end + PW_KT - 1) / PW_KT;
            n_act = lim_wave_max > 0 ? (lim_wave_max + PW_KT - 1) / PW_KT : 0;
        }
        __syncthreads();                                   // (s_range is used again below)
    }
    if (DENSE) {
        mrow = (const T*)p.mask + (int64_t)b * p.m_sb + (int64_t)hq * p.m_sh + (int64_t)min(my_i, Sq - 1) * p.m_si;
        // (a wavefront whose 32 rows lie past Sq computes nothing; its flag reads stay inside the array on the last row block)
        mflags = mask_flags_of(p, b, hq) + (int64_t)min((q0 >> 5) + wave, ((Sq + 31) >> 5) - 1) * ((Skv + 31) >> 5);
        int lo = 0x7fffffff, hi = -1;
        for (int t = lane; t < n_act; t += 64)
            if (mflags[t] != 2) { lo = min(lo, t); hi = max(hi, t); }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            lo = min(lo, __shfl_xor(lo, off, 64));
            hi = max(hi, __shfl_xor(hi, off, 64));
        }
        w_first = __builtin_amdgcn_readfirstlane(hi < 0 ? 0 : lo);
        n_act = __builtin_amdgcn_readfirstlane(hi + 1);
        if (lane == 0) { s_range[wave] = hi < 0 ? 0x7fffffff : lo; s_range[4 + wave] = hi; }
        __syncthreads();
        int g_lo = s_range[0], g_hi = s_range[4];
#pragma unroll
        for (int w2 = 1; w2 < 4; ++w2) { g_lo = min(g_lo, s_range[w2]); g_hi = max(g_hi, s_range[4 + w2]); }
        // (uniform by construction; said explicitly, because tile numbers end up in scalar copy descriptors)
        t_first = __builtin_amdgcn_readfirstlane(g_hi < 0 ? 0 : g_lo);
        n_tiles = __builtin_amdgcn_readfirstlane(g_hi + 1);      // (0 when the mask hides everything from these 128 rows)
    }

    // ---- global -> LDS copy plan: wavefront-wide load ii = wave * LPW + c fills LDS bytes [ii * 1024, +1024) of a tile ----
    int k_voff[LPW], v_voff[LPW];
#pragma unroll
    for (int c = 0; c < LPW; ++c) {
        const int pos = (wave * LPW + c) * 64 + lane;
        const int row = pos / L::CPR, slot = pos % L::CPR;
        k_voff[c] = dma_chunk_offset(row, (int)p.k_ss * 2, slot ^ L::fk(row), p.D * 2);
        v_voff[c] = dma_chunk_offset(row, (int)p.v_ss * 2, slot ^ L::fv(row), p.Dv * 2);
    }
    const int64_t k_tile_bytes = (int64_t)PW_KT * p.k_ss * 2, v_tile_bytes = (int64_t)PW_KT * p.v_ss * 2;
    auto issue = [&](const T* base, int64_t tile_bytes, int64_t row_stride, int row_elems, int t, int buf, const int (&voff)[LPW]) __attribute__((always_inline)) {
        // bytes to the end of the last row this workgroup may see: loads past that return 0 (rows past a batch entry's
        // key count are never read)
        int64_t rem = (int64_t)(j_end - t * PW_KT - 1) * row_stride * 2 + row_elems * 2;
        if (rem > 0x7fffffffLL) rem = 0x7fffffffLL;
        const uint4v r = dma_descriptor((const char*)base + t * tile_bytes, (int)rem);
        const unsigned dst = lds_address(smem) + buf * TILE + wave * LPW * 1024;
#pragma unroll
        for (int c = 0; c < LPW; ++c) dma_copy16(r, dst + c * 1024, voff[c]);
    };
    auto issue_kv = [&](int t) __attribute__((always_inline)) {
        issue(kp, k_tile_bytes, p.k_ss, p.D, t, t & 1, k_voff);
        issue(vp, v_tile_bytes, p.v_ss, p.Dv, t, 2 + (t & 1), v_voff);
    };
    if (n_tiles > t_first) issue_kv(t_first);
    int flag_next = 1;      // the flag of the next tile, read one tile ahead
    if (DENSE && n_tiles > t_first) flag_next = mflags[t_first];

    // ---- operands ----------------------------------------------------------------------------------------------
    // Q^T (B operand, resident): this lane's row, elements 16 s + 8 g .. + 7 of it per k-step s (beyond D: zeros, like K's).
    // Fetched 16 bytes per lane, eight lanes to a run of a row, and brought into that layout through this wavefront's 4 KiB
    // of the K buffer the first copies do not fill (nothing is copied there before the loop's first barrier).
    vec8 qreg[NSTEP];
    {
        uint4v qraw[NSTEP / 4][4];
        fetch_q_rows(qraw, qp, q0 + wave * 32, Sq, p.q_ss, p.D, lane);
        stage_q_rows(qreg, qraw, smem + ((t_first + 1) & 1) * TILE + wave * 4096, lane);
        // scale * log2(e) folded into Q once (rounded back to the storage type, as sdpa_prefill_mfma.hip does): the product
        // then yields the scores in the log2 units the softmax works in, whatever the sign of the scale
        const float c2 = p.scale * 1.4426950408889634f;
#pragma unroll
        for (int s = 0; s < NSTEP; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) qreg[s][e] = (T)((float)qreg[s][e] * c2);
    }
    // K operand of k-step s: row ql, logical chunk 2 s + g, stored at chunk (2 s + g) ^ fk(ql) = (g ^ fk(ql)) ^ 2 s; the
    // row's offset and the chunk bits share none, so the address is k_base ^ (s << 5).
    const int k_base = ql * L::ROWB + ((g ^ L::fk(ql)) << 4);
    // V operand (transposing read) of column block db, half h: the 16 lanes of a group fetch a 4-key x 16-d patch (lane n:
    // key n / 4, d 4 (n % 4) .. + 3).  Row 8 h + 4 g + n / 4, logical chunk 4 db + 2 dh + (n % 4) / 2 at chunk
    // ^ fv(row) = ^ 4 (n / 4): v_base[h] ^ (db << 6).
    int v_base[2];
    {
        const int n = lane & 15, dh = (lane >> 4) & 1;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int r = 8 * h + 4 * g + (n >> 2);
            const int chunk = 2 * dh + ((n & 3) >> 1);
            v_base[h] = r * L::ROWB + ((chunk ^ L::fv(r)) << 4) + (n & 1) * 8;
        }
    }

    float m_run = -INFINITY, l_run = 0.0f;
    floatx16 o_acc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[db][r] = 0.0f;

    for (int t = t_first; t < n_tiles; ++t) {
        // K(t), V(t) have arrived for everyone, everyone is done with tile t - 1: its buffers take tile t + 1
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (t + 1 < n_tiles) issue_kv(t + 1);
        int flag = 1;
        if (DENSE) {      // (arrived with the tile: the wait above covers it)
            flag = __builtin_amdgcn_readfirstlane(flag_next);
            if (t + 1 < n_tiles) flag_next = mflags[t + 1];
        }
        if (t >= n_act || t < w_first) continue;      // nothing of this tile is visible to the wavefront's rows
        const char* kb = smem + (t & 1) * TILE;
        const char* vb = smem + (2 + (t & 1)) * TILE;
        const int j0 = t * PW_KT;
        // ---- S^T = K Q^T ----
        floatx16 sacc;
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[r] = 0.0f;
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
            const vec8 a = *(const vec8*)(kb + (k_base ^ (s << 5)));
            sacc = Mma<T>::run(a, qreg[s], sacc);
        }
        // (the order asked of the scheduler: K reads four matrix instructions ahead of their use: + 4 - 8 %)
        __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
        for (int i = 0; i < NSTEP - 4; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        // register r is key j0 + 8 (r / 4) + 4 g + (r % 4)
        if (DENSE && flag != 1) {      // the mask's values of this lane's 16 keys (no registers to spare for asking earlier)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const int j = j0 + 8 * r4 + 4 * g;
                typedef T vec4 __attribute__((ext_vector_type(4)));
                // (rows of the mask are contiguous and 8-byte aligned here - the host sends other masks elsewhere; keys at and
                // beyond Skv are hidden by the limits below whatever is added to them)
                vec4 m4 = {(T)0.0f, (T)0.0f, (T)0.0f, (T)0.0f};
                if (j + 3 < Skv) m4 = *(const vec4*)(mrow + j);
                else if (j < Skv) {      // the group that straddles the last key: its keys below Skv one by one
#pragma unroll
                    for (int e = 0; e < 4; ++e) m4[e] = mrow[min(j + e, Skv - 1)];
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) sacc[4 * r4 + e] = __builtin_fmaf((float)m4[e], 1.4426950408889634f, sacc[4 * r4 + e]);
            }
        }
        if (j0 + PW_KT > lim_wave_min) {                  // (uniform) the tile crosses a limit of this wavefront
            const int rel = lim_lane - (j0 + 4 * g);
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (8 * (r / 4) + (r % 4) >= rel) sacc[r] = -INFINITY;
        }
        float tmax = sacc[0];
#pragma unroll
        for (int r = 1; r < 16; ++r) tmax = fmaxf(tmax, sacc[r]);
        tmax = xor32_max(tmax);
        // the reference moves only when a tile's maximum passes it by more than 2^8 (or the row sees its first key)
        const bool need = tmax > m_run + PF_RESCALE_THRESHOLD;
        if (__builtin_amdgcn_ballot_w64(need) != 0) {
            const float alpha = need ? __builtin_amdgcn_exp2f(m_run - tmax) : 1.0f;      // (first key: exp2(-inf) = 0 times 0)
            if (need) m_run = tmax;
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) o_acc[db][r] *= alpha;
        }
        const float m_use = (m_run == -INFINITY) ? 0.0f : m_run;
        // P^T in storage precision: element e of k-step ks is register 8 ks + e; the denominator is summed from the rounded values
        vec8 pb[2];
        float rsum = 0.0f;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int e = 0; e < 8; ++e) pb[ks][e] = (T)__builtin_amdgcn_exp2f(sacc[8 * ks + e] - m_use);
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                typename Mma<T>::vec2 pr = {pb[ks][e], pb[ks][e + 1]};
                rsum = Mma<T>::add2(pr, rsum);
            }
        }
        l_run += rsum;
        // ---- O^T += V^T P^T ----
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int db = 0; db < NDB; ++db) {
                short8v av;
                av.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4v __attribute__((address_space(3)))*)(vb + ks * 16 * L::ROWB + (v_base[0] ^ (db << 6))));
                av.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4v __attribute__((address_space(3)))*)(vb + ks * 16 * L::ROWB + (v_base[1] ^ (db << 6))));
                o_acc[db] = Mma<T>::run(__builtin_bit_cast(vec8, av), pb[ks], o_acc[db]);
            }
        // (V reads - two per matrix instruction - four matrix instructions ahead)
        __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
        for (int i = 0; i < 2 * NDB - 4; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
    }

    // ---- normalise and store --------------------------------------------------------------------------------------
    const float l_tot = xor32_sum(l_run);
    if constexpr (SPLIT) {
        // partial result of this split: unnormalised O, and (reference, sum) in the log2 units the combine kernel takes for 16-bit
        // storage; a row that saw no key in this split says so with a reference of -inf
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
                p.ws_ml[slot * 2 + 0] = l_tot == 0.0f ? -INFINITY : m_run;
                p.ws_ml[slot * 2 + 1] = l_tot;
            }
        }
        return;
    }
    const float inv = (l_tot == 0.0f) ? __builtin_nanf("") : 1.0f / l_tot;      // no visible key: NaN, as the reference
    if (my_i < rows_b && p.lse && g == 0)       // m_run and the sum are in log2 units of the scaled scores
        p.lse[((int64_t)b * p.Hq + hq) * Sq + my_i] = l_tot == 0.0f ? -INFINITY : (m_run + __builtin_log2f(l_tot)) * 0.6931471805599453f;
    // through this wavefront's 4 KiB of the K buffer the last tile did not use: every wavefront is past the barrier of that
    // tile, i.e. done with the tile before it, and nothing has been copied since
    store_o_rows(o_acc, inv, smem + (n_tiles & 1) * TILE + wave * 4096, op, q0 + wave * 32, rows_b, p.o_ss, p.Dv, lane);
#endif
}

// Host has validated: dtype f16 / bf16, 128 < max(D, Dv) <= 256 in whole 16-byte vectors, finite scale; with a dense mask its
// block flags have been written (launch_mask_classify);
// rows 16-byte aligned with unit last-dim stride, row strides below 2^24 elements.
hipError_t launch_sdpa_combine(const SdpaParams& p, int dtype, hipStream_t stream);

hipError_t launch_sdpa_prefill_wide(const SdpaParams& p0, int dtype, hipStream_t stream)
{
    SdpaParams p = p0;
    const int nqb = (p.Sq + PF_BM - 1) / PF_BM;
    const int64_t total = (int64_t)nqb * p.Hq * p.B;
    if (total <= 0) return hipSuccess;
    if (total > 0x7fffffffLL) return hipErrorInvalidValue;
    // two workgroups per compute unit, an eighth of the compute units per XCD
    p.interleave = work_interleave(p.causal != 0 || p.mask != nullptr, 2 * device_cus() / 8, p.G, nqb, (total & 7) == 0 ? total >> 3 : total);
    p.deal_groups = (total & 7) == 0 ? work_deal(p.interleave, p.G, nqb, total >> 3, p.causal != 0 || p.mask != nullptr) : 0;
    if (p.mask && p.mask_lims) {       // the blocks whose rows all have a limit; then, below, the others
        if (dtype == 1) hipLaunchKernelGGL((sdpa_prefill_wide_kernel<f16_t, 2>), dim3((unsigned)total), dim3(256), 0, stream, p);
        else hipLaunchKernelGGL((sdpa_prefill_wide_kernel<bf16_t, 2>), dim3((unsigned)total), dim3(256), 0, stream, p);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (!p.mask && p.num_splits > 1) {       // split launch: partial results, then the split-KV kernels' combine pass
        const dim3 grid((unsigned)total, (unsigned)p.num_splits);
        if (dtype == 1) hipLaunchKernelGGL((sdpa_prefill_wide_kernel<f16_t, 0, true>), grid, dim3(256), 0, stream, p);
        else hipLaunchKernelGGL((sdpa_prefill_wide_kernel<bf16_t, 0, true>), grid, dim3(256), 0, stream, p);
        hipError_t e = hipGetLastError();
        return e != hipSuccess ? e : launch_sdpa_combine(p, dtype, stream);
    }
    if (p.mask) {
        if (dtype == 1) hipLaunchKernelGGL((sdpa_prefill_wide_kernel<f16_t, 1>), dim3((unsigned)total), dim3(256), 0, stream, p);
        else hipLaunchKernelGGL((sdpa_prefill_wide_kernel<bf16_t, 1>), dim3((unsigned)total), dim3(256), 0, stream, p);
    } else if (dtype == 1) hipLaunchKernelGGL((sdpa_prefill_wide_kernel<f16_t, 0>), dim3((unsigned)total), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((sdpa_prefill_wide_kernel<bf16_t, 0>), dim3((unsigned)total), dim3(256), 0, stream, p);
    return hipGetLastError();
}

}  // namespace incin_rocm
