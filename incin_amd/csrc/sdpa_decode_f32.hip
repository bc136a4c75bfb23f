// Split-KV attention for the query rows that share one key/value head, in IEEE single precision on the gfx950 matrix
// cores (v_mfma_f32_16x16x4_f32: f32 operands, products and sums), head dimensions up to 256 (instances for 64, 128 and
// 256; a smaller D or Dv is zero-padded on the way into LDS): grouped-query decode and short
// runs of query rows over a long f32 cache - f32 being the one dtype the reference's own operator runs end to end
// (crates/incin-backends/src/cpu/ops/shape_ops.rs:1245-1269), with a 1e-5 bar.  The vector-ALU split-KV kernel
// handles one to a few rows per KV head at the memory system's rate and then runs out of arithmetic; the prefill kernel
// launches one workgroup per 128 rows, which for a decode step is a handful of workgroups walking the whole cache.
//
// Design: that of sdpa_decode_mfma.hip, which see - one workgroup (4 wavefronts) per (batch, KV head, chunk of 16 or 32
// rows, split), the split's keys dealt to the wavefronts in blocks of one 8 KiB slot (16 keys at D = 128, 32 at D = 64),
// each wavefront streaming its blocks through its own ring of LDS slots (non-temporal global -> LDS copies, constant
// wait), no barrier in the loop, one meeting of the four wavefronts' (maximum, sum, O^T) at the end; same partial-result
// format, same combine kernel.  What differs is the instruction and with it the layouts:
//
//   S^T = K Q'^T     16 keys x 16 rows per instruction, summed over four values of d: lane (n = lane % 16, g = lane / 16)
//                    supplies K[key n][d] and Q'[row n][d] for the d its group holds.  Which four is free as long as
//                    both operands agree, so a lane reads four consecutive floats d = 16 j + 4 g .. + 3 (one 16-byte
//                    LDS read) and they serve four instructions.  In the 16 x 16 result a lane owns ONE row (column n)
//                    and four keys (register r is key 4 g + r): maxima and sums are in-lane plus two lane exchanges.
//   O^T += V^T P^T   that accumulator layout is already the B-operand layout of the second product - register r is the
//                    k-step of keys 4 g + r - and the A operand is V[4 g + r][16 db + n]: a 4-byte LDS read of 16
//                    consecutive floats of one row per quarter-wavefront; no transposition, no conversion.
//
// The matrix pipe is not far from a bound here: an instruction takes 32 cycles and a block of 16 keys x 16 rows needs
// D of them, i.e. a compute unit turns over 16 KiB of cache per 2048 D / 128 cycles per 16 rows - 19 TB/s over the device at
// 16 rows, 9.6 TB/s at 32 - so 32 rows per workgroup is where the cache is read once; more rows go in chunks of 32.
#include <cstdlib>

#include "sdpa_decode_ring.h"

namespace incin_rocm {

typedef float floatx4 __attribute__((ext_vector_type(4)));

// lanes l, l ^ 16, l ^ 32, l ^ 48 (the four lanes of a query row) end with the maximum / the sum of their values
__device__ __forceinline__ float quad_max(float x)
{
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    return xor32_max(x);
}
__device__ __forceinline__ float quad_sum(float x)
{
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    return xor32_sum(x);
}

//
// LIMS: the launch is one half of a request with a mask tensor (one query head per KV head, or whole 128-row blocks per head):
// mask_row_limits_kernel wrote, per mask row, n if the row is n zeros and then -inf, else -1.  A workgroup whose 128-row
// block of rows all have a limit takes the limits - the tensor says nothing more - and the others leave at once: the f32
// prefill kernel's dense-mask launch that follows computes those, and leaves the blocks computed here alone.
template <int D, int NSLOT, int NRB, bool LIMS = false>
__global__ __launch_bounds__(256) void sdpa_decode_f32_kernel(SdpaParams p)
{
#if defined(__HIP_DEVICE_COMPILE__)
    typedef F32Layout<D> L;
    constexpr int NJ = D / 16;                         // groups of four k-steps of the S^T product
    constexpr int NDB = D / 16;                        // 16-wide blocks of the head dimension
    constexpr int NDBW = NDB / 4;                      // of which a wavefront stores this many at the end
    constexpr int SLOT = D > 128 ? 2 * DM_SLOT_BYTES : DM_SLOT_BYTES;      // a slot holds 8 KiB, at D = 256 the 16 KiB of 16 keys
    constexpr int BLOCK = SLOT / L::ROWB;              // keys per block: 16 (D = 128, 256), 32 (D = 64)
    constexpr int KB = BLOCK / 16;                     // 16-key sub-blocks of a block
    constexpr int CPB = SLOT / 1024;                   // wavefront-wide 1 KiB copies per block
    constexpr int CHUNK = 16 * NRB;                    // rows per workgroup
    constexpr float LN2 = 0.6931471805599453f;
    extern __shared__ __attribute__((aligned(1024))) char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ql = lane & 15, g = lane >> 4;
    const int Sq = p.Sq, Skv = p.Skv;
    const int R = p.G * Sq;
    const int nchunks = (R + CHUNK - 1) / CHUNK;
    const int split = blockIdx.x;
    int hkv, chunk_id;
    int b;
    decode_work_item(nchunks, (p.causal || LIMS) && p.G == 1, NSLOT == 2, &b, &hkv, &chunk_id);
    const int r0 = chunk_id * CHUNK;

    int kv_len = Skv;
    if (p.kv_lens) kv_len = clampi(p.kv_lens[b], 0, Skv);
    const int k_begin = split * p.split_len;

    // this lane's rows, one per block of 16 (the four lanes l % 16 share them), and the keys each may see inside this split
    bool valid[NRB];
    int hq[NRB], qi[NRB], lim[NRB];
    int lim_hi = 0, lim_lo = 0x7fffffff;
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb) {
        const int row = r0 + 16 * rb + ql;
        valid[rb] = row < R;
        const int gq = valid[rb] ? row / Sq : 0;
        qi[rb] = valid[rb] ? row % Sq : 0;
        hq[rb] = hkv * p.G + gq;
        int l = min(k_begin + p.split_len, kv_len);
        if (p.causal) l = min(l, causal_limit(qi[rb], Sq, Skv));
        lim[rb] = valid[rb] ? l : 0;
    }
    if (LIMS) {
        // the 128-row block of this chunk's query head (rows of a chunk share a head: the host sends no other launches here)
        __shared__ int s_ok[4];
        const int head_row0 = (r0 / Sq) * Sq, i0 = r0 - head_row0;
        const int blk0 = (i0 / 128) * 128, blk1 = min(blk0 + 128, Sq);
        const int32_t* lims = mask_lims_of(p, b, hkv * p.G + r0 / Sq);
        bool ok = true;
        for (int i = blk0 + tid; i < blk1; i += 256) ok = ok && lims[p.m_si ? i : 0] >= 0;
        const bool wave_ok = __builtin_amdgcn_ballot_w64(!ok) == 0;
        if (lane == 0) s_ok[wave] = wave_ok ? 1 : 0;
        __syncthreads();
        if ((s_ok[0] & s_ok[1] & s_ok[2] & s_ok[3]) == 0) return;      // (uniform) the dense-mask launch computes this block
#pragma unroll
        for (int rb = 0; rb < NRB; ++rb)
            if (valid[rb]) lim[rb] = min(lim[rb], lims[p.m_si ? qi[rb] : 0]);
    }
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb) {
        lim_hi = max(lim_hi, lim[rb]);
        if (valid[rb]) lim_lo = min(lim_lo, lim[rb]);
    }
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) {
        lim_hi = max(lim_hi, __shfl_xor(lim_hi, off, 64));
        lim_lo = min(lim_lo, __shfl_xor(lim_lo, off, 64));
    }
    const int k_end = __builtin_amdgcn_readfirstlane(lim_hi);          // rows at and beyond are never read
    const int mask_from = __builtin_amdgcn_readfirstlane(lim_lo);      // blocks that end at or before need no mask
    const int n_blocks = k_end > k_begin ? (k_end - k_begin + BLOCK - 1) / BLOCK : 0;
    const int my_blocks = n_blocks > wave ? (n_blocks - wave + 3) >> 2 : 0;      // blocks wave, wave + 4, ...

    // ---- global -> LDS copy plan (whole rows; 16-byte chunk c of row r lands at chunk c ^ f(r)) -----------------------
    int k_voff[CPB], v_voff[CPB];
#pragma unroll
    for (int c = 0; c < CPB; ++c) {
        const int pos = c * 64 + lane;
        const int r = pos / L::CPR, slot = pos % L::CPR;
        k_voff[c] = dma_chunk_offset(r, (int)p.k_ss * 4, slot ^ L::f(r), p.D * 4);
        v_voff[c] = dma_chunk_offset(r, (int)p.v_ss * 4, slot ^ L::f(r), p.Dv * 4);
    }
    const float* kp = (const float*)p.k + (int64_t)b * p.k_sb + (int64_t)hkv * p.k_sh;
    const float* vp = (const float*)p.v + (int64_t)b * p.v_sb + (int64_t)hkv * p.v_sh;
    // The copies of this wavefront go K(block 0) V(0) K(1) V(1) ...; copy number n lands in slot n % NSLOT.  Address of
    // the next block of each tensor and the bytes from there to the end of row k_end - 1 (loads past that deliver
    // zeros: what an unwritten cache tail holds never enters LDS).
    const int64_t k_step = (int64_t)4 * BLOCK * p.k_ss * 4, v_step = (int64_t)4 * BLOCK * p.v_ss * 4;
    const int first_key = k_begin + wave * BLOCK;
    const char* k_next = (const char*)kp + (int64_t)first_key * p.k_ss * 4;
    const char* v_next = (const char*)vp + (int64_t)first_key * p.v_ss * 4;
    int64_t k_rem = (int64_t)(k_end - first_key - 1) * p.k_ss * 4 + p.D * 4;
    int64_t v_rem = (int64_t)(k_end - first_key - 1) * p.v_ss * 4 + p.Dv * 4;
    // bytes a descriptor may cover: none once the tensor's blocks are used up, 2^31 - 1 at most
    auto clamp31 = [](int64_t x) __attribute__((always_inline)) {
        const unsigned hi = (unsigned)((unsigned long long)x >> 32), lo = (unsigned)x;
        return x <= 0 ? 0 : (hi | (lo >> 31)) != 0 ? 0x7fffffff : (int)lo;
    };
    const unsigned ring = lds_address(smem) + wave * NSLOT * SLOT;
    // Copies are started unconditionally, NSLOT ahead of their use: past the wavefront's last block the descriptor
    // covers nothing, such a copy fetches nothing and delivers zeros into a slot nobody reads any more - which keeps the
    // count of copies in flight, and with it the wait for the oldest, the same from the first block to the last.
    int issued = 0, slot_in = 0;
    auto issue_next = [&]() __attribute__((always_inline)) {
        // The slot about to be refilled was read by this wavefront's LDS loads just before: those loads have delivered
        // once lgkmcnt is 0 (the "memory" clobber keeps them above this point in program order).
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        const unsigned dst = ring + slot_in * SLOT;
        if ((issued & 1) == 0) {
            const uint4v rk = dma_descriptor(k_next, clamp31(k_rem));
#pragma unroll
            for (int c = 0; c < CPB; ++c) dm_copy16(rk, dst + c * 1024, k_voff[c]);
            k_next += k_step;
            k_rem -= k_step;
        } else {
            const uint4v rv = dma_descriptor(v_next, clamp31(v_rem));
#pragma unroll
            for (int c = 0; c < CPB; ++c) dm_copy16(rv, dst + c * 1024, v_voff[c]);
            v_next += v_step;
            v_rem -= v_step;
        }
        ++issued;
        slot_in = slot_in + 1 == NSLOT ? 0 : slot_in + 1;
    };
    // ---- operands ----------------------------------------------------------------------------------------------
    // Q'^T = (Q * scale * log2 e)^T (B operand, resident): this lane's row, floats 16 j + 4 g .. + 3 of it per group j.  All of
    // its loads are asked for first, every lane from an address that exists (a lane beyond the head dimension reads the row's
    // start, a row that does not exist is row 0 of the group's first head), and nothing looks at them until the first copies
    // are on their way too: a load that is scaled right behind its issue waits for itself, one after the other, and behind
    // the copies for all of those as well.
    floatx4 qreg[NRB][NJ];
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb) {
        const float* qrow = (const float*)p.q + (int64_t)b * p.q_sb + (int64_t)hq[rb] * p.q_sh + (int64_t)qi[rb] * p.q_ss;
#pragma unroll
        for (int j = 0; j < NJ; ++j) qreg[rb][j] = *(const floatx4*)(qrow + (j * 16 + g * 4 < p.D ? j * 16 + g * 4 : 0));
    }
    for (int u = 0; u < NSLOT; ++u) issue_next();
    __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0), told to the compiler too: the Q rows (and the first copies) have arrived
    asm volatile("" ::: "memory");
    {
        const float c2 = p.scale * 1.4426950408889634f;      // scores in log2 units
#pragma unroll
        for (int rb = 0; rb < NRB; ++rb)
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const bool in = valid[rb] && j * 16 + g * 4 < p.D;      // (rows that do not exist, and beyond the head dimension: zeros, like K's)
#pragma unroll
                for (int e = 0; e < 4; ++e) qreg[rb][j][e] = in ? qreg[rb][j][e] * c2 : 0.0f;
            }
    }
    // K operand of group j: row n of the sub-block, logical chunk 4 j + g, stored at chunk (4 j + g) ^ f(n) = (g ^ f(n)) ^ 4 j;
    // the row's offset, the chunk bits of g ^ f and those of 4 j share no bits, so the address is k_base ^ (j << 6).
    const int k_base = ql * L::ROWB + ((g ^ L::f(ql)) << 4);
    // V operand of k-step r, block db: row 4 g + r of the sub-block, float 16 db + n, i.e. logical chunk 4 db + n / 4 at
    // chunk ((n / 4) ^ f(4 g + r)) ^ 4 db: v_base[r] ^ (db << 6).
    int v_base[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) v_base[r] = (4 * g + r) * L::ROWB + (((ql >> 2) ^ L::f(4 * g + r)) << 4) + (ql & 3) * 4;

    float m_run[NRB], l_run[NRB];
    floatx4 o_acc[NRB][NDB];
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb) {
        m_run[rb] = -INFINITY;
        l_run[rb] = 0.0f;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) o_acc[rb][db][r] = 0.0f;
    }

    int slot_out = 0;              // slot of the copy consumed next
    for (int jb = 0; jb < my_blocks; ++jb) {
        const int j0 = first_key + jb * 4 * BLOCK;
        // ---- S^T = K Q'^T: two chains over the halves of the head dimension ----
        wait_oldest_copy<NSLOT, CPB>();
        const char* kb = smem + (wave * NSLOT + slot_out) * SLOT;
        slot_out = slot_out + 1 == NSLOT ? 0 : slot_out + 1;
        floatx4 s0[NRB][KB], s1[NRB][KB];
#pragma unroll
        for (int rb = 0; rb < NRB; ++rb)
#pragma unroll
            for (int kb2 = 0; kb2 < KB; ++kb2)
#pragma unroll
                for (int r = 0; r < 4; ++r) { s0[rb][kb2][r] = 0.0f; s1[rb][kb2][r] = 0.0f; }
        // The block's K operands, in the order the products take them.  With one wavefront per SIMD nobody else covers
        // the latency of an LDS read, so the reads run two steps ahead of the matrix instructions that use them (the
        // order is asked of the scheduler below, which would otherwise fetch each pair only when its registers come free).
        floatx4 ka[KB][NJ];
#pragma unroll
        for (int j = 0; j < NJ / 2; ++j)
#pragma unroll
            for (int kb2 = 0; kb2 < KB; ++kb2) {
                ka[kb2][j] = *(const floatx4*)(kb + kb2 * 16 * L::ROWB + (k_base ^ (j << 6)));
                ka[kb2][j + NJ / 2] = *(const floatx4*)(kb + kb2 * 16 * L::ROWB + (k_base ^ ((j + NJ / 2) << 6)));
            }
#pragma unroll
        for (int j = 0; j < NJ / 2; ++j)
#pragma unroll
            for (int kb2 = 0; kb2 < KB; ++kb2)
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int rb = 0; rb < NRB; ++rb) {
                        s0[rb][kb2] = __builtin_amdgcn_mfma_f32_16x16x4f32(ka[kb2][j][e], qreg[rb][j][e], s0[rb][kb2], 0, 0, 0);
                        s1[rb][kb2] = __builtin_amdgcn_mfma_f32_16x16x4f32(ka[kb2][j + NJ / 2][e], qreg[rb][j + NJ / 2][e], s1[rb][kb2], 0, 0, 0);
                    }
        {
            constexpr int STEPS = (NJ / 2) * KB;      // each: two LDS reads, 8 NRB matrix instructions
            __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
            for (int i = 0; i < STEPS - 2; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 4 * NRB, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 4 * NRB, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, 16 * NRB, 0);
        }
        issue_next();              // (the block's values are in registers: its slot takes the next copy)
        // register r of sub-block kb2 is key j0 + 16 kb2 + 4 g + r
        const bool masked = j0 + BLOCK > mask_from;
        floatx4 pr[NRB][KB];
#pragma unroll
        for (int rb = 0; rb < NRB; ++rb) {
#pragma unroll
            for (int kb2 = 0; kb2 < KB; ++kb2)
#pragma unroll
                for (int r = 0; r < 4; ++r) pr[rb][kb2][r] = s0[rb][kb2][r] + s1[rb][kb2][r];
            if (masked) {
                const int rel = lim[rb] - (j0 + 4 * g);
#pragma unroll
                for (int kb2 = 0; kb2 < KB; ++kb2)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (16 * kb2 + r >= rel) pr[rb][kb2][r] = -INFINITY;
            }
            float tmax = pr[rb][0][0];
#pragma unroll
            for (int kb2 = 0; kb2 < KB; ++kb2)
#pragma unroll
                for (int r = 0; r < 4; ++r) tmax = fmaxf(tmax, pr[rb][kb2][r]);
            tmax = quad_max(tmax);               // largest score of the row in this block (log2 units)
            // The reference the probabilities are taken against moves only when a block's maximum passes it by more
            // than 2^8 (or the row sees its first key): exact in exact arithmetic, probabilities stay <= 2^8, and O^T
            // is rescaled on the first block and then hardly ever.
            const bool need = tmax > m_run[rb] + PF_RESCALE_THRESHOLD;      // (-inf + 8 = -inf: any finite maximum passes it)
            if (__builtin_amdgcn_ballot_w64(need) != 0) {
                const float alpha = need ? __builtin_amdgcn_exp2f(m_run[rb] - tmax) : 1.0f;   // (first key: exp2(-inf) = 0 times 0)
                if (need) m_run[rb] = tmax;
                l_run[rb] *= alpha;
#pragma unroll
                for (int db = 0; db < NDB; ++db)
#pragma unroll
                    for (int r = 0; r < 4; ++r) o_acc[rb][db][r] *= alpha;
            }
            const float m_use = (m_run[rb] == -INFINITY) ? 0.0f : m_run[rb];
            float rsum = 0.0f;
#pragma unroll
            for (int kb2 = 0; kb2 < KB; ++kb2)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    pr[rb][kb2][r] = __builtin_amdgcn_exp2f(pr[rb][kb2][r] - m_use);
                    rsum += pr[rb][kb2][r];
                }
            l_run[rb] += rsum;
        }
        // ---- O^T += V^T P^T ----
        wait_oldest_copy<NSLOT, CPB>();
        const char* vb = smem + (wave * NSLOT + slot_out) * SLOT;
        slot_out = slot_out + 1 == NSLOT ? 0 : slot_out + 1;
#pragma unroll
        for (int kb2 = 0; kb2 < KB; ++kb2)
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int db = 0; db < NDB; ++db) {
                    const float vv = *(const float*)(vb + kb2 * 16 * L::ROWB + (v_base[r] ^ (db << 6)));
#pragma unroll
                    for (int rb = 0; rb < NRB; ++rb) o_acc[rb][db] = __builtin_amdgcn_mfma_f32_16x16x4f32(vv, pr[rb][kb2][r], o_acc[rb][db], 0, 0, 0);
                }
        {
            constexpr int READS = 4 * NDB * KB;       // each feeds NRB matrix instructions; the reads run eight ahead
            __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
            for (int i = 0; i < READS - 8; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, NRB, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, 8 * NRB, 0);
        }
        issue_next();
    }

    // ---- the four wavefronts' results meet (the rings are done with) --------------------------------------------------
    float* s_m = (float*)smem;                               // [4][CHUNK] maxima
    float* s_l = s_m + 4 * CHUNK;                            // [4][CHUNK] sums, rescaled
    float* s_o = s_l + 4 * CHUNK;                            // [4 wavefronts][NRB][NDB][4][64] O^T registers, rescaled
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");         // (the empty copies started past the last block too)
    __syncthreads();
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb)
        if (g == 0) s_m[wave * CHUNK + 16 * rb + ql] = m_run[rb];
    __syncthreads();
    float M[NRB];
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb) {
        M[rb] = s_m[16 * rb + ql];
#pragma unroll
        for (int w = 1; w < 4; ++w) M[rb] = fmaxf(M[rb], s_m[w * CHUNK + 16 * rb + ql]);
        const float M_use = (M[rb] == -INFINITY) ? 0.0f : M[rb];
        const float f = __builtin_amdgcn_exp2f(m_run[rb] - M_use);
        const float l_w = quad_sum(l_run[rb]) * f;
        if (g == 0) s_l[wave * CHUNK + 16 * rb + ql] = l_w;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) s_o[(((wave * NRB + rb) * NDB + db) * 4 + r) * 64 + lane] = o_acc[rb][db][r] * f;
    }
    __syncthreads();
    // ---- this wavefront's NDBW blocks of 16 columns of every row: lane (n, g) holds floats 16 db + 4 g .. + 3 of row n ----
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb) {
        if (!valid[rb]) continue;
        float l_tot = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) l_tot += s_l[w * CHUNK + 16 * rb + ql];
        const float inv = (l_tot == 0.0f) ? __builtin_nanf("") : 1.0f / l_tot;      // no visible key: NaN, as the reference
        const int64_t slot = (((int64_t)b * p.Hq + hq[rb]) * Sq + qi[rb]) * p.num_splits + split;
#pragma unroll
        for (int d2 = 0; d2 < NDBW; ++d2) {
            const int db = wave * NDBW + d2;
            floatx4 o = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int w = 0; w < 4; ++w)
#pragma unroll
                for (int r = 0; r < 4; ++r) o[r] += s_o[(((w * NRB + rb) * NDB + db) * 4 + r) * 64 + lane];
            if (p.num_splits == 1) {
                float* orow = (float*)p.o + (int64_t)b * p.o_sb + (int64_t)hq[rb] * p.o_sh + (int64_t)qi[rb] * p.o_ss;
#pragma unroll
                for (int r = 0; r < 4; ++r) o[r] *= inv;
                if (16 * db + 4 * g < p.Dv) *(floatx4*)(orow + 16 * db + 4 * g) = o;
            } else {
                *(floatx4*)(p.ws_acc + slot * D + 16 * db + 4 * g) = o;
            }
        }
        if (wave == 0 && g == 0) {
            if (p.num_splits == 1) {
                if (p.lse)      // the row's softmax normaliser, natural log (M and the sum are in log2 units)
                    p.lse[((int64_t)b * p.Hq + hq[rb]) * Sq + qi[rb]] = l_tot == 0.0f ? -INFINITY : (M[rb] + __builtin_log2f(l_tot)) * LN2;
            } else {
                p.ws_ml[slot * 2 + 0] = M[rb] * LN2;      // natural-log units, as the combine kernel takes them for f32 storage
                p.ws_ml[slot * 2 + 1] = l_tot;
            }
        }
    }
#endif
}

hipError_t launch_sdpa_combine(const SdpaParams& p, int dtype, hipStream_t stream);

template <int D, int NSLOT, int NRB, bool LIMS = false>
static hipError_t launch_decode_f32_t(const SdpaParams& p, hipStream_t stream)
{
    // the rings, or what the wavefronts' results need when they meet at the end, whichever is more
    constexpr size_t slot_bytes = D > 128 ? 2 * DM_SLOT_BYTES : DM_SLOT_BYTES;
    constexpr size_t ring_bytes = (size_t)4 * NSLOT * slot_bytes, merge_bytes = (size_t)NRB * (4 * 16 * 2 + 4 * (D / 16) * 4 * 64) * sizeof(float);
    constexpr size_t lds = ring_bytes > merge_bytes ? ring_bytes : merge_bytes;
    auto kern = sdpa_decode_f32_kernel<D, NSLOT, NRB, LIMS>;
    // the dynamic-LDS limit of this instance is raised once per device, not per launch
    static std::atomic<uint64_t> prepared{0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    const uint64_t bit = 1ull << (dev & 63);
    if (!(prepared.load(std::memory_order_acquire) & bit)) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        prepared.fetch_or(bit, std::memory_order_release);
    }
    const int R = p.G * p.Sq;
    const int nchunks = (R + 16 * NRB - 1) / (16 * NRB);
    dim3 grid(p.num_splits, p.Hkv * nchunks, p.B);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, p);
    return hipGetLastError();
}

// Rows a workgroup of the f32 kernel takes: 16, or 32 (two blocks of 16 against the same K and V operands) when more than
// 16 rows share a KV head.
int decode_f32_chunk_rows(int R) { return R > 16 ? 32 : 16; }

// Host has validated: f32, D and Dv <= 128 in whole 16-byte vectors (p.Dp = the instance), rows 16-byte aligned with unit last-dim stride, row strides below 2^22
// elements, split_len a multiple of 256 (whole rounds of the four wavefronts' blocks of 16 or 32 keys).
template <int D>
static hipError_t launch_decode_f32_d(const SdpaParams& p, bool two_slots, hipStream_t stream)
{
    // 32 rows: always the two-slot rings, two workgroups per compute unit - one wavefront per SIMD leaves nothing to cover a
    // wavefront's start-up, softmax and waits (measured against five slots on prefill and decode shapes alike: level to 1.3
    // times ahead, config 2 of the benchmark 65 -> 51 us)
    if (decode_f32_chunk_rows(p.G * p.Sq) == 32) return launch_decode_f32_t<D, 2, 2>(p, stream);
    return two_slots ? launch_decode_f32_t<D, 2, 1>(p, stream) : launch_decode_f32_t<D, DM_NSLOT, 1>(p, stream);
}

// two_slots: the two-slot rings (two workgroups per compute unit) for the 16-row form, as the launcher of the 16-bit kernel
// chooses them for short splits.
hipError_t launch_sdpa_decode_f32(const SdpaParams& p, bool two_slots, hipStream_t stream)
{
    hipError_t e;
    // head dimensions above 128: two slots of 16 KiB (a block of 16 keys) per wavefront, 16 or 32 rows
    if (p.Dp == 256) e = decode_f32_chunk_rows(p.G * p.Sq) == 32 ? launch_decode_f32_t<256, 2, 2>(p, stream) : launch_decode_f32_t<256, 2, 1>(p, stream);
    else e = p.Dp == 128 ? launch_decode_f32_d<128>(p, two_slots, stream) : launch_decode_f32_d<64>(p, two_slots, stream);
    if (e != hipSuccess || p.num_splits == 1) return e;
    return launch_sdpa_combine(p, 0, stream);
}

// The row-limit half of an f32 request with a mask tensor (see the kernel): 32 rows per workgroup, one split, no combine
// pass.  Host has validated what launch_sdpa_decode_f32 asks for, one query head per KV head or S_q a multiple of 128, D and
// Dv <= 128, and p.mask_lims written.
hipError_t launch_sdpa_decode_f32_limits(const SdpaParams& p, hipStream_t stream)
{
    return p.Dp == 128 ? launch_decode_f32_t<128, 2, 2, true>(p, stream) : launch_decode_f32_t<64, 2, 2, true>(p, stream);
}

}  // namespace incin_rocm
