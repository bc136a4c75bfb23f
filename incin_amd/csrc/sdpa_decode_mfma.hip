// Split-KV attention for the query rows that share one key/value head, on the gfx950 matrix cores (f16 / bf16,
// head dimensions up to 256: instances for 64, 128 and 256, a smaller D or Dv zero-padded on the way into LDS): grouped-query decode, where the vector-ALU split-KV kernel runs out of arithmetic (it spends
// ~24 vector instructions per query row on every 2 KiB of cache it reads), and short runs of query rows over a long
// cache.  Same function as the other attention kernels (crates/incin-backends/src/cpu/ops/shape_ops.rs:1245-1269),
// same partial-result format as the vector-ALU split-KV kernel, same combine kernel.
//
// The work is bound by the bandwidth of the cache reads, so the design serves the memory system first:
//
//   * one workgroup (4 wavefronts) per (batch, KV head, chunk of 32 or 64 query rows, split), one workgroup per compute
//     unit (two of the two-slot form that short splits take: see the launcher).  The split's keys are dealt to the wavefronts in blocks of 32 (D = 64: 64; wavefront w takes blocks w, w + 4, ...), and
//     a wavefront works through its blocks on its own: no barrier in the loop, nothing shared.  Each wavefront owns a
//     ring of NSLOT 8 KiB slots in LDS that the K and V blocks pass through in the order they are needed
//     (K0 V0 K1 V1 ...), filled straight from global memory (buffer_load ... lds, whole rows, 1 KiB per instruction);
//     a slot is refilled the moment its block has been used, so NSLOT - 1 blocks per wavefront - 128 KiB per compute
//     unit with five slots - are in flight at any time, and the wait for the oldest copy is a constant s_waitcnt: copies
//     past a wavefront's last block are started all the same, with a descriptor that covers nothing;
//   * 32 rows are the 32 columns of S^T = K Q^T (v_mfma_f32_32x32x16, a lane owns one row's scores of the block; rows
//     that do not exist are zero columns - matrix throughput is not what is scarce here), the softmax is the usual
//     online one per wavefront, and O^T += V^T P^T takes V through transposing LDS reads; with 64 rows every K and V
//     operand read from LDS serves two such products;
//   * at the end the four wavefronts' (maximum, sum, O^T) meet once in LDS (the rings are done with by then) and
//     wavefront w writes columns 32 w .. 32 w + 31 of every row.
//
// Rows: row r of a chunk is (query head hkv * G + r / Sq, position r % Sq) - the G heads of the group times the Sq
// positions.  The scale is applied to the f32 scores (any sign), masks as -inf before the maximum.
//
// A dense additive mask (MASK instances; the reference's mask tensor: crates/incin-backends/src/cpu/ops/shape_ops.rs:
// 1262-1266; unit key stride, 16-byte aligned rows, Skv a multiple of 8) is added to the scaled scores.  Its values take
// the road the keys take: copied global -> LDS a block ahead (two copies of 64 x 16 bytes per 32 rows x 32 keys, into one
// of two small buffers per wavefront behind the rings), read from there when the block's scores are ready.  The copies
// share the counter of memory operations in flight with the ring's, so the wait for them is a count as well: three ring
// copies and the next block's mask copies have been issued since - which asks of the ring only that the copy it needs
// next anyway has landed.  (Loading the values into registers would leave the waiting to the compiler, which knows
// nothing of the ring's copies and would drain it at every block.)
#include <cstdlib>

#include "sdpa_decode_ring.h"

namespace incin_rocm {

template <typename T, int D, int NSLOT, int NRB, bool MASK = false>
__global__ __launch_bounds__(256) void sdpa_decode_mfma_kernel(SdpaParams p)
{
#if defined(__HIP_DEVICE_COMPILE__)
    typedef typename Mma<T>::vec8 vec8;
    typedef PfLayout<D> L;
    constexpr int NSTEP = D / 16, NDB = D / 32;
    constexpr int SLOT = D > 128 ? 2 * DM_SLOT_BYTES : DM_SLOT_BYTES;      // a slot holds 8 KiB, at D = 256 the 16 KiB of 32 keys
    constexpr int KB = SLOT / (32 * L::ROWB);          // 32-key sub-blocks of a block: 2 at D = 64, else 1
    constexpr int BLOCK = 32 * KB;                     // keys per block
    constexpr int CPB = SLOT / 1024;                   // wavefront-wide 1 KiB copies per block
    constexpr int NDBW = NDB >= 4 ? NDB / 4 : 1;       // 32-wide blocks of the head dimension a wavefront stores at the end
    extern __shared__ __attribute__((aligned(1024))) char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ql = lane & 31, g = lane >> 5;
    const int Sq = p.Sq, Skv = p.Skv;
    const int R = p.G * Sq;
    constexpr int CHUNK = 32 * NRB;                    // rows per workgroup
    const int nchunks = (R + CHUNK - 1) / CHUNK;
    const int split = blockIdx.x;
    int hkv, chunk_id;
    int b;
    decode_work_item(nchunks, p.causal && p.G == 1, NSLOT == 2, &b, &hkv, &chunk_id);
    const int r0 = chunk_id * CHUNK;

    int kv_len = Skv;
    if (p.kv_lens) kv_len = clampi(p.kv_lens[b], 0, Skv);
    const int k_begin = split * p.split_len;

    // this lane's rows, one per block of 32 (lanes l and l + 32 share them), and the keys each may see inside this split
    bool valid[NRB];
    int hq[NRB], qi[NRB], lim[NRB];
    int lim_hi = 0, lim_lo = 0x7fffffff;
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb) {
        const int row = r0 + 32 * rb + ql;
        valid[rb] = row < R;
        const int gq = valid[rb] ? row / Sq : 0;
        qi[rb] = valid[rb] ? row % Sq : 0;
        hq[rb] = hkv * p.G + gq;
        int l = min(k_begin + p.split_len, kv_len);
        if (p.causal) l = min(l, causal_limit(qi[rb], Sq, Skv));
        lim[rb] = valid[rb] ? l : 0;
        lim_hi = max(lim_hi, lim[rb]);
        if (valid[rb]) lim_lo = min(lim_lo, l);
    }
#pragma unroll
    for (int off = 16; off >= 1; off >>= 1) {
        lim_hi = max(lim_hi, __shfl_xor(lim_hi, off, 64));
        lim_lo = min(lim_lo, __shfl_xor(lim_lo, off, 64));
    }
    const int k_end = __builtin_amdgcn_readfirstlane(lim_hi);          // rows at and beyond are never read
    const int mask_from = __builtin_amdgcn_readfirstlane(lim_lo);      // blocks that end at or before need no mask
    const int n_blocks = k_end > k_begin ? (k_end - k_begin + BLOCK - 1) / BLOCK : 0;
    const int my_blocks = n_blocks > wave ? (n_blocks - wave + 3) >> 2 : 0;      // blocks wave, wave + 4, ...

    // ---- global -> LDS copy plan (rows of 256 bytes, chunk slot c ^ f(row) as in the prefill kernels' tiles) ---------
    int k_voff[CPB], v_voff[CPB];
#pragma unroll
    for (int c = 0; c < CPB; ++c) {
        const int pos = c * 64 + lane;
        const int r = pos / L::CPR, slot = pos % L::CPR;
        k_voff[c] = dma_chunk_offset(r, (int)p.k_ss * 2, slot ^ L::fk(r), p.D * 2);
        v_voff[c] = dma_chunk_offset(r, (int)p.v_ss * 2, slot ^ L::fv(r), p.Dv * 2);
    }
    const T* kp = (const T*)p.k + (int64_t)b * p.k_sb + (int64_t)hkv * p.k_sh;
    const T* vp = (const T*)p.v + (int64_t)b * p.v_sb + (int64_t)hkv * p.v_sh;
    // The copies of this wavefront go K(block 0) V(0) K(1) V(1) ...; copy number n lands in slot n % NSLOT.  Address of
    // the next block of each tensor and the bytes from there to the end of row k_end - 1 (loads past that deliver
    // zeros: what an unwritten cache tail holds never enters LDS).
    const int64_t k_step = (int64_t)4 * BLOCK * p.k_ss * 2, v_step = (int64_t)4 * BLOCK * p.v_ss * 2;
    const int first_key = k_begin + wave * BLOCK;
    const char* k_next = (const char*)kp + (int64_t)first_key * p.k_ss * 2;
    const char* v_next = (const char*)vp + (int64_t)first_key * p.v_ss * 2;
    int64_t k_rem = (int64_t)(k_end - first_key - 1) * p.k_ss * 2 + p.D * 2;
    int64_t v_rem = (int64_t)(k_end - first_key - 1) * p.v_ss * 2 + p.Dv * 2;
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
    // Q^T (B operand, resident): this lane's row, elements 16 s + 8 g .. + 7 of it per k-step s.  All of its loads are asked
    // for first, every lane from an address that exists (a lane beyond the head dimension reads the row's start, a row that
    // does not exist is row 0 of the group's first head), and nothing looks at them until the first copies are on their way
    // too: a load that is looked at right behind its issue waits for itself, eight of them one after the other, and behind
    // the copies for all of those as well.
    vec8 qreg[NRB][NSTEP];
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb) {
        const T* qrow = (const T*)p.q + (int64_t)b * p.q_sb + (int64_t)hq[rb] * p.q_sh + (int64_t)qi[rb] * p.q_ss;
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) qreg[rb][s] = *(const vec8*)(qrow + (s * 16 + g * 8 < p.D ? s * 16 + g * 8 : 0));
    }
    for (int u = 0; u < NSLOT; ++u) issue_next();
    __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0), told to the compiler too: the Q rows (and the first copies) have arrived
    asm volatile("" ::: "memory");
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb)
#pragma unroll
        for (int s = 0; s < NSTEP; ++s)
            if (!valid[rb] || s * 16 + g * 8 >= p.D)      // (rows that do not exist, and beyond the head dimension: zeros, like K's)
#pragma unroll
                for (int e = 0; e < 8; ++e) qreg[rb][s][e] = (T)0.0f;
    // K operand: lane (ql, g) reads row ql, logical chunk 2 s + g
    int k_addr[NSTEP];
    {
        const int F = L::fk(ql);
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) k_addr[s] = ql * L::ROWB + (((2 * s + g) ^ F) << 4);
    }
    // V operand (transposing read): the 16 lanes of a group fetch a 4-key x 16-d patch (lane n: key n / 4,
    // d 4 (n % 4) .. + 3) and receive (d = n, keys 0 .. 3).  Row within a 16-row block: 8 h + 4 g + n / 4; logical chunk
    // 4 db + 2 dh + (n % 4) / 2.
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

    // dense mask: two buffers per wavefront behind the rings, each NRB x KB tiles of 32 rows x 32 keys (64 bytes per row; the
    // 16-byte chunk c of row r at chunk c ^ (r / 4 % 4), which spreads the reads of a chunk down 32 rows over the banks).
    // Copy c (of two per tile) brings rows 16 c + lane / 4, chunk lane % 4: the lane's offsets into the mask are those rows'.
    constexpr int MTILE = 2048, MBUF = NRB * KB * MTILE, NMC = NRB * KB * 2;      // bytes per tile / buffer, copies per block
    [[maybe_unused]] const unsigned mzone = lds_address(smem) + 4 * NSLOT * SLOT + wave * 2 * MBUF;
    [[maybe_unused]] int m_voff[NRB][2];
    [[maybe_unused]] uint4v m_desc = {0u, 0u, 0u, 0u};
    if constexpr (MASK) {
#pragma unroll
        for (int rb = 0; rb < NRB; ++rb)
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const int rr = 16 * c + (lane >> 2), row = r0 + 32 * rb + rr;
                const int hq_r = hkv * p.G + (row < R ? row / Sq : 0), qi_r = row < R ? row % Sq : 0;
                m_voff[rb][c] = (int)(((int64_t)hq_r * p.m_sh + (int64_t)qi_r * p.m_si) * 2) + ((((lane & 3) ^ ((rr >> 2) & 3))) << 4);
            }
        // everything from this batch entry's first mask byte to the last one any row reaches; chunks beyond arrive as zeros
        // (they belong to keys past Skv in the last row, which the limits hide)
        const int64_t extent = ((p.m_sh ? (int64_t)(p.Hq - 1) * p.m_sh : 0) + (p.m_si ? (int64_t)(Sq - 1) * p.m_si : 0) + Skv) * 2;
        m_desc = dma_descriptor((const T*)p.mask + (int64_t)b * p.m_sb, (int)(extent > 0x7fffffffLL ? 0x7fffffffLL : extent));
    }
    // the mask's values for the block of this wavefront that starts at key jb, into buffer `buf`
    [[maybe_unused]] auto issue_mask = [&](int jb, int buf) __attribute__((always_inline)) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");      // (the buffer's last readers have their values)
#pragma unroll
        for (int rb = 0; rb < NRB; ++rb)
#pragma unroll
            for (int kb2 = 0; kb2 < KB; ++kb2)
#pragma unroll
                for (int c = 0; c < 2; ++c)
                    dma_copy16_at(m_desc, mzone + buf * MBUF + (rb * KB + kb2) * MTILE + c * 1024, m_voff[rb][c], (jb + 32 * kb2) * 2);
    };
    if constexpr (MASK) {
        issue_mask(first_key, 0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // (start-up: the first block's values, with the first copies)
    }

    const float sc2 = p.scale * 1.4426950408889634f;      // scores in log2 units
    float m_run[NRB], l_run[NRB];
    floatx16 o_acc[NRB][NDB];
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb) {
        m_run[rb] = -INFINITY;
        l_run[rb] = 0.0f;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) o_acc[rb][db][r] = 0.0f;
    }

    int slot_out = 0;              // slot of the copy consumed next
    for (int j = 0; j < my_blocks; ++j) {
        const int j0 = first_key + j * 4 * BLOCK;
        // the mask's values of this wavefront's next block start towards the buffer the block before this one used
        if constexpr (MASK) issue_mask(j0 + 4 * BLOCK, (j + 1) & 1);
        // ---- S^T = K Q^T ----
        wait_oldest_copy<NSLOT, CPB>();
        const char* kb = smem + (wave * NSLOT + slot_out) * SLOT;
        slot_out = slot_out + 1 == NSLOT ? 0 : slot_out + 1;
        floatx16 sacc[NRB][KB];
#pragma unroll
        for (int rb = 0; rb < NRB; ++rb)
#pragma unroll
            for (int kb2 = 0; kb2 < KB; ++kb2)
#pragma unroll
                for (int r = 0; r < 16; ++r) sacc[rb][kb2][r] = 0.0f;
#pragma unroll
        for (int s = 0; s < NSTEP; ++s)
#pragma unroll
            for (int kb2 = 0; kb2 < KB; ++kb2) {
                const vec8 a = *(const vec8*)(kb + k_addr[s] + kb2 * 32 * L::ROWB);
#pragma unroll
                for (int rb = 0; rb < NRB; ++rb) sacc[rb][kb2] = Mma<T>::run(a, qreg[rb][s], sacc[rb][kb2]);
            }
        issue_next();              // (the block's values are in registers: its slot takes the next copy)
        // register r of sub-block kb2 is key j0 + 32 kb2 + 8 (r / 4) + 4 g + (r % 4)
        const bool masked = j0 + BLOCK > mask_from;
        vec8 pb[NRB][2 * KB];
        if constexpr (MASK) {
            // issued since this block's mask copies: two ring copies in the last iteration, the next block's mask copies and
            // one ring copy in this one - everything older has landed once no more than that is in flight
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * CPB + NMC) : "memory");
        }
#pragma unroll
        for (int rb = 0; rb < NRB; ++rb) {
#pragma unroll
            for (int kb2 = 0; kb2 < KB; ++kb2)
#pragma unroll
                for (int r = 0; r < 16; ++r) sacc[rb][kb2][r] *= sc2;
            if constexpr (MASK) {
                // registers 4 r4 .. 4 r4 + 3 of sub-block kb2 are keys 8 r4 + 4 g .. + 3 of it: half g of chunk r4 of row ql
                const char* mt = smem + 4 * NSLOT * SLOT + wave * 2 * MBUF + (j & 1) * MBUF + rb * KB * MTILE;
#pragma unroll
                for (int kb2 = 0; kb2 < KB; ++kb2)
#pragma unroll
                    for (int r4 = 0; r4 < 4; ++r4) {
                        typedef T vec4 __attribute__((ext_vector_type(4)));
                        const vec4 mv = *(const vec4*)(mt + kb2 * MTILE + ql * 64 + ((r4 ^ ((ql >> 2) & 3)) << 4) + g * 8);
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            sacc[rb][kb2][4 * r4 + e] = __builtin_fmaf((float)mv[e], 1.4426950408889634f, sacc[rb][kb2][4 * r4 + e]);
                    }
            }
            if (masked) {
                const int rel = lim[rb] - (j0 + 4 * g);
#pragma unroll
                for (int kb2 = 0; kb2 < KB; ++kb2)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        if (32 * kb2 + 8 * (r / 4) + (r % 4) >= rel) sacc[rb][kb2][r] = -INFINITY;
            }
            float tmax = sacc[rb][0][0];
#pragma unroll
            for (int kb2 = 0; kb2 < KB; ++kb2)
#pragma unroll
                for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, sacc[rb][kb2][r]);
            tmax = xor32_max(tmax);              // largest score of the row in this block (log2 units)
            // The reference the probabilities are taken against moves only when a block's maximum passes it by more
            // than 2^8 (or the row sees its first key): exact in exact arithmetic, probabilities stay <= 2^8, and O^T -
            // 64 accumulator registers - is rescaled on the first block and then hardly ever.
            const bool need = tmax > m_run[rb] + PF_RESCALE_THRESHOLD;      // (-inf + 8 = -inf: any finite maximum passes it)
            if (__builtin_amdgcn_ballot_w64(need) != 0) {
                const float alpha = need ? __builtin_amdgcn_exp2f(m_run[rb] - tmax) : 1.0f;   // (first key: exp2(-inf) = 0 times 0)
                if (need) m_run[rb] = tmax;
                l_run[rb] *= alpha;
#pragma unroll
                for (int db = 0; db < NDB; ++db)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o_acc[rb][db][r] *= alpha;
            }
            const float m_use = (m_run[rb] == -INFINITY) ? 0.0f : m_run[rb];
            // P^T in storage precision: element e of k-step ks is register 8 (ks % 2) + e of sub-block ks / 2; the
            // denominator is summed from the rounded values
            float rsum = 0.0f;
#pragma unroll
            for (int ks = 0; ks < 2 * KB; ++ks) {
#pragma unroll
                for (int e = 0; e < 8; ++e) pb[rb][ks][e] = (T)__builtin_amdgcn_exp2f(sacc[rb][ks / 2][8 * (ks % 2) + e] - m_use);
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    typename Mma<T>::vec2 pr = {pb[rb][ks][e], pb[rb][ks][e + 1]};
                    rsum = Mma<T>::add2(pr, rsum);
                }
            }
            l_run[rb] += rsum;
        }
        // ---- O^T += V^T P^T ----
        wait_oldest_copy<NSLOT, CPB>();
        const char* vb = smem + (wave * NSLOT + slot_out) * SLOT;
        slot_out = slot_out + 1 == NSLOT ? 0 : slot_out + 1;
#pragma unroll
        for (int ks = 0; ks < 2 * KB; ++ks)
#pragma unroll
            for (int db = 0; db < NDB; ++db) {
                short8v av;
                av.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4v __attribute__((address_space(3)))*)(vb + v_addr[db][0] + ks * 16 * L::ROWB));
                av.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4v __attribute__((address_space(3)))*)(vb + v_addr[db][1] + ks * 16 * L::ROWB));
#pragma unroll
                for (int rb = 0; rb < NRB; ++rb) o_acc[rb][db] = Mma<T>::run(__builtin_bit_cast(vec8, av), pb[rb][ks], o_acc[rb][db]);
            }
        issue_next();
    }

    // ---- the four wavefronts' results meet (the rings are done with) --------------------------------------------------
    float* s_m = (float*)smem;                               // [4][CHUNK] maxima
    float* s_l = s_m + 4 * CHUNK;                            // [4][CHUNK] sums, rescaled
    float* s_o = s_l + 4 * CHUNK;                            // [4 wavefronts][NRB][NDB][16][64] O^T registers, rescaled
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");         // (the empty copies started past the last block too)
    __syncthreads();
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb)
        if (g == 0) s_m[wave * CHUNK + 32 * rb + ql] = m_run[rb];
    __syncthreads();
    float M[NRB];
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb) {
        M[rb] = s_m[32 * rb + ql];
#pragma unroll
        for (int w = 1; w < 4; ++w) M[rb] = fmaxf(M[rb], s_m[w * CHUNK + 32 * rb + ql]);
        const float M_use = (M[rb] == -INFINITY) ? 0.0f : M[rb];
        const float f = __builtin_amdgcn_exp2f(m_run[rb] - M_use);
        const float l_w = xor32_sum(l_run[rb]) * f;
        if (g == 0) s_l[wave * CHUNK + 32 * rb + ql] = l_w;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) s_o[(((wave * NRB + rb) * NDB + db) * 16 + r) * 64 + lane] = o_acc[rb][db][r] * f;
    }
    __syncthreads();
    // ---- this wavefront's NDBW blocks of 32 columns of every row (D = 64: the first two wavefronts' one) --------------
    if (wave * NDBW >= NDB) return;
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb) {
        if (!valid[rb]) continue;
        float l_tot = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) l_tot += s_l[w * CHUNK + 32 * rb + ql];
        const float inv = (l_tot == 0.0f) ? __builtin_nanf("") : 1.0f / l_tot;      // no visible key: NaN, as the reference
        const int64_t slot = (((int64_t)b * p.Hq + hq[rb]) * Sq + qi[rb]) * p.num_splits + split;
#pragma unroll
        for (int d2 = 0; d2 < NDBW; ++d2) {
            const int db = wave * NDBW + d2;
            floatx16 o;
#pragma unroll
            for (int r = 0; r < 16; ++r) o[r] = 0.0f;
#pragma unroll
            for (int w = 0; w < 4; ++w)
#pragma unroll
                for (int r = 0; r < 16; ++r) o[r] += s_o[(((w * NRB + rb) * NDB + db) * 16 + r) * 64 + lane];
            if (p.num_splits == 1) {
                T* orow = (T*)p.o + (int64_t)b * p.o_sb + (int64_t)hq[rb] * p.o_sh + (int64_t)qi[rb] * p.o_ss + 32 * db + 4 * g;
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    typedef T vec4 __attribute__((ext_vector_type(4)));
                    vec4 w;
#pragma unroll
                    for (int e = 0; e < 4; ++e) w[e] = (T)(o[r4 * 4 + e] * inv);
                    if (32 * db + 4 * g + r4 * 8 < p.Dv) *(vec4*)(orow + r4 * 8) = w;
                }
            } else {
                float* arow = p.ws_acc + slot * D + 32 * db + 4 * g;
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    typedef float f4 __attribute__((ext_vector_type(4)));
                    f4 w = {o[r4 * 4], o[r4 * 4 + 1], o[r4 * 4 + 2], o[r4 * 4 + 3]};
                    *(f4*)(arow + r4 * 8) = w;
                }
            }
        }
        if (wave == 0 && g == 0) {
            if (p.num_splits == 1) {
                if (p.lse)      // the row's softmax normaliser, natural log (M and the sum are in log2 units)
                    p.lse[((int64_t)b * p.Hq + hq[rb]) * Sq + qi[rb]] = l_tot == 0.0f ? -INFINITY : (M[rb] + __builtin_log2f(l_tot)) * 0.6931471805599453f;
            } else {
                p.ws_ml[slot * 2 + 0] = M[rb];      // log2 units, as the combine kernel takes them for 16-bit storage
                p.ws_ml[slot * 2 + 1] = l_tot;
            }
        }
    }
#endif
}

hipError_t launch_sdpa_combine(const SdpaParams& p, int dtype, hipStream_t stream);

template <typename T, int D, int NSLOT, int NRB, bool MASK = false>
static hipError_t launch_decode_mfma_t(const SdpaParams& p, hipStream_t stream)
{
    // the rings (and behind them, with a dense mask, two buffers of its values per wavefront), or what the wavefronts'
    // results need when they meet at the end, whichever is more
    constexpr size_t slot_bytes = D > 128 ? 2 * DM_SLOT_BYTES : DM_SLOT_BYTES;
    constexpr size_t mask_bytes = MASK ? (size_t)4 * 2 * NRB * (slot_bytes / (32 * D * 2)) * 2048 : 0;
    constexpr size_t ring_bytes = (size_t)4 * NSLOT * slot_bytes + mask_bytes, merge_bytes = (size_t)NRB * (4 * 32 * 2 + 4 * (D / 32) * 16 * 64) * sizeof(float);
    constexpr size_t lds = ring_bytes > merge_bytes ? ring_bytes : merge_bytes;
    static_assert(lds <= 160 * 1024, "a compute unit's LDS");
    auto kern = sdpa_decode_mfma_kernel<T, D, NSLOT, NRB, MASK>;
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
    const int nchunks = (R + 32 * NRB - 1) / (32 * NRB);
    dim3 grid(p.num_splits, p.Hkv * nchunks, p.B);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, p);
    return hipGetLastError();
}

int decode_f32_chunk_rows(int R);
hipError_t launch_sdpa_decode_f32(const SdpaParams& p, bool two_slots, hipStream_t stream);

// Rows a workgroup takes: 32, or 64 (two blocks of 32 against the same K and V operands) when more than 32 rows share a KV
// head - the cache is then read once for 64 rows instead of once per 32.  (f32, dtype 0: 16 or 32, sdpa_decode_f32.hip.)
int decode_mfma_chunk_rows(int R, int dtype, int d_pad) { return dtype == 0 ? decode_f32_chunk_rows(R) : R > 32 && d_pad <= 128 ? 64 : 32; }

// Workgroups a compute unit holds at a time: two of the two-slot form (one block of rows, splits of up to DM_SHORT_KEYS
// keys of 16-bit storage or half as many of f32), one otherwise.  The planner fills rounds of this many.
int decode_mfma_workgroups_per_cu(int chunk_rows, int64_t split_len, int dtype, int d_pad)
{
    if (d_pad > 128) return 1;
    if (dtype == 0) return chunk_rows == 32 || 2 * split_len <= DM_SHORT_KEYS ? 2 : 1;      // (f32, 32 rows: always two-slot rings)
    return chunk_rows == 32 && split_len <= DM_SHORT_KEYS ? 2 : 1;
}

// INCIN_ROCM_DECODE_SLOTS = 2 or 5 overrides the choice between the two forms of the one-block kernels (for tests: both
// forms on any shape).
static bool decode_two_slots(const SdpaParams& p, int dtype)
{
    const char* forced = getenv("INCIN_ROCM_DECODE_SLOTS");
    const int slots = forced ? atoi(forced) : 0;
    const int one_block = dtype == 0 ? 16 : 32;
    return slots == 2 || (slots != DM_NSLOT && decode_mfma_workgroups_per_cu(one_block, p.split_len, dtype, p.Dp) == 2);
}

// With a dense mask: the same forms with four slots per wavefront instead of five (the mask's buffers take the room); 64 rows
// per workgroup at D = 64 do not fit and are not offered (the planner sends such launches elsewhere).
template <typename T, int D>
static hipError_t launch_decode_mfma_masked(const SdpaParams& p, hipStream_t stream)
{
    if constexpr (D <= 128) {
        if (decode_mfma_chunk_rows(p.G * p.Sq, 2, D) == 64) {
            if constexpr (D == 128) return launch_decode_mfma_t<T, D, 4, 2, true>(p, stream);
            else return hipErrorInvalidValue;
        }
        if (decode_two_slots(p, 2)) return launch_decode_mfma_t<T, D, 2, 1, true>(p, stream);
        return launch_decode_mfma_t<T, D, 4, 1, true>(p, stream);
    } else {
        return launch_decode_mfma_t<T, D, 2, 1, true>(p, stream);
    }
}

// Host has validated: dtype f16 / bf16, D and Dv <= 128 in whole 16-byte vectors (p.Dp = the instance), rows 16-byte aligned with unit last-dim stride, row strides
// below 2^24 elements, split_len a multiple of 256 (whole rounds of the four wavefronts' blocks of 32 or 64 keys).
template <typename T, int D>
static hipError_t launch_decode_mfma_d(const SdpaParams& p, hipStream_t stream)
{
    if (p.mask) return launch_decode_mfma_masked<T, D>(p, stream);
    if (decode_mfma_chunk_rows(p.G * p.Sq, 2, D) == 64) return launch_decode_mfma_t<T, D, DM_NSLOT, 2>(p, stream);
    // Short splits (up to DM_SHORT_KEYS keys: 16 blocks per wavefront) take rings of two slots, which lets a compute
    // unit hold two workgroups: with so little to stream, what counts is that one workgroup's start-up (its first
    // copies' latency) and end (the wavefronts' results meeting, the stores) overlap another's arithmetic.  Measured
    // on launches of 268 MB of cache, two slots against five: 256-key splits 73 against 46 % of the memory bandwidth,
    // 512: 81 / 63, 1024: 80 / 73, 2048: 87.5 / 86.3; 4096: 78.5 / 80 (one sequence of 131072 keys); 8192: 84 / 86.7.
    if (decode_two_slots(p, 2)) return launch_decode_mfma_t<T, D, 2, 1>(p, stream);
    return launch_decode_mfma_t<T, D, DM_NSLOT, 1>(p, stream);
}

hipError_t launch_sdpa_decode_mfma(const SdpaParams& p, int dtype, hipStream_t stream)
{
    if (dtype == 0) return launch_sdpa_decode_f32(p, decode_two_slots(p, 0), stream);
    hipError_t e;
    // head dimensions above 128: one form - 32 rows, two slots of 16 KiB (a block of 32 keys) per wavefront
    if (p.Dp == 256 && p.mask) e = dtype == 1 ? launch_decode_mfma_masked<f16_t, 256>(p, stream) : launch_decode_mfma_masked<bf16_t, 256>(p, stream);
    else if (p.Dp == 256) e = dtype == 1 ? launch_decode_mfma_t<f16_t, 256, 2, 1>(p, stream) : launch_decode_mfma_t<bf16_t, 256, 2, 1>(p, stream);
    else if (p.Dp == 128) e = dtype == 1 ? launch_decode_mfma_d<f16_t, 128>(p, stream) : launch_decode_mfma_d<bf16_t, 128>(p, stream);
    else e = dtype == 1 ? launch_decode_mfma_d<f16_t, 64>(p, stream) : launch_decode_mfma_d<bf16_t, 64>(p, stream);
    if (e != hipSuccess || p.num_splits == 1) return e;
    return launch_sdpa_combine(p, dtype, stream);
}

}  // namespace incin_rocm
