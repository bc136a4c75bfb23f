// bf16 / f16 attention forward on the gfx950 matrix cores, software-pipelined
// inside each wavefront (prefill shapes).
//
// Mathematics, operand layouts, LDS swizzle and the global->LDS path are those
// of sdpa_prefill_mfma.hip (see there).  What differs is the schedule.  On this
// hardware MFMA and vector-ALU instructions overlap only when they come from
// the SAME wavefront, so each wavefront keeps three key half-tiles (32 keys) in
// flight and every half-iteration u issues, interleaved in one instruction
// stream:
//
//     matrix pipe :  S^T(u+1) = K(u+1) Q^T   then   O^T += V^T(u-1) P^T(u-1)
//     vector ALU  :  P(u) = exp2(S(u) c - m), row sum;  then max S(u+1)
//
// All three pieces are independent of one another.  Scores and probabilities
// alternate between two register sets by half-tile parity, so no register is
// ever copied.  One 64-key K/V tile (two half-tiles) is loaded per barrier,
// one tile ahead, into two alternating LDS stages, exactly as in the
// un-pipelined kernel: K(t) is read by half-iterations 2t-1 and 2t, V(t) by
// 2t+1 and 2t+2, and the barrier that opens tile step t publishes K(t), V(t-1).
//
// Running maximum: the maximum of S(u+1) is known one half-iteration before
// P(u+1) is formed.  If it exceeds the reference maximum m by more than 2^8 the
// lane raises m at once (and rescales its running sum); the accumulator O is
// rescaled one half-iteration later, after the pending product with P(u), which
// was formed against the old m, has been added.  Otherwise m stays stale, which
// is exact in exact arithmetic and keeps every probability <= 2^8.
#include <type_traits>

#include "sdpa_mfma_common.h"

namespace incin_rocm {

template <int V> using ic = std::integral_constant<int, V>;

template <typename T, int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void sdpa_prefill_pipe_kernel(SdpaParams p)
{
#if defined(__HIP_DEVICE_COMPILE__)   // the body uses device-only types (buffer descriptors); the host pass needs only the stub
    typedef typename Mma<T>::vec8 vec8;
    typedef PfLayout<D> L;
    constexpr int NQ = D / 16;             // MFMAs of one S^T half-tile (k-steps over the head dimension)
    constexpr int NDB = D / 32;            // 32-wide blocks of the head dimension
    constexpr int NP = 2 * NDB;            // MFMAs of one O^T half-tile update (2 k-steps of 16 keys x NDB blocks)
    constexpr int NSLOT = NQ + NP;
    constexpr int LPW = L::LOADS_PER_WAVE;
    constexpr int TILE = L::TILE_BYTES;
    constexpr int HALF = 32 * L::ROWB;     // bytes from half-tile 0 to half-tile 1 inside a tile

    __shared__ __attribute__((aligned(1024))) char smem[4 * TILE];   // K stage 0, K stage 1, V stage 0, V stage 1

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);     // wavefront-uniform by construction: keep it scalar
    const int ql = lane & 31, g = lane >> 5;
    const int Sq = p.Sq, Skv = p.Skv;

    // ---- which (batch, head, query block) -----------------------------------
    // Workgroups reach the 8 XCDs round-robin by id; hand each XCD a contiguous
    // range of the work list so heads that share K/V stay in one L2, and order
    // each head's query blocks longest-first.
    const int nqb = (Sq + PF_BM - 1) / PF_BM;
    const int total = gridDim.x;
    int vid = blockIdx.x;
    if ((total & 7) == 0) vid = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);
    const int gq = vid % p.G;
    const int qb = nqb - 1 - (vid / p.G) % nqb;
    const int bhkv = vid / (p.G * nqb);
    const int hkv = bhkv % p.Hkv, b = bhkv / p.Hkv;
    const int hq = hkv * p.G + gq;
    const int q0 = qb * PF_BM;

    const T* qp = (const T*)p.q + (int64_t)b * p.q_sb + (int64_t)hq * p.q_sh;
    const T* kp = (const T*)p.k + (int64_t)b * p.k_sb + (int64_t)hkv * p.k_sh;
    const T* vp = (const T*)p.v + (int64_t)b * p.v_sb + (int64_t)hkv * p.v_sh;
    T* op = (T*)p.o + (int64_t)b * p.o_sb + (int64_t)hq * p.o_sh;

    int kv_len = Skv;
    if (p.kv_lens) kv_len = clampi(p.kv_lens[b], 0, Skv);
    const int coff = Skv - Sq;
    int j_end = kv_len;                    // keys visible to the workgroup
    const int my_i = q0 + wave * 32 + ql;
    int lim_lane = kv_len, lim_wave_min = kv_len;   // keys visible to this lane's query / to every query of the wavefront
    if (p.causal) {
        const int last_row = min(q0 + PF_BM - 1, Sq - 1);
        j_end = clampi(last_row + coff + 1, 0, kv_len);
        lim_lane = clampi(my_i + coff + 1, 0, kv_len);
        lim_wave_min = clampi(q0 + wave * 32 + coff + 1, 0, kv_len);
    }
    const int N = (j_end + PF_BN - 1) / PF_BN;      // 64-key tiles of the workgroup

    // ---- global -> LDS copy plan ---------------------------------------------------
    // wavefront-wide load number ii = wave*LPW + c fills LDS bytes [ii*1024, ii*1024 + 1024)
    // of a tile; lane -> position ii*64 + lane -> (row, slot) -> global chunk slot ^ f(row).
    int k_voff[LPW], v_voff[LPW];
#pragma unroll
    for (int c = 0; c < LPW; ++c) {
        const int pos = (wave * LPW + c) * 64 + lane;
        const int row = pos / L::CPR, slot = pos % L::CPR;
        k_voff[c] = row * (int)p.k_ss * 2 + (slot ^ L::fk(row)) * 16;
        v_voff[c] = row * (int)p.v_ss * 2 + (slot ^ L::fv(row)) * 16;
    }
    const int64_t k_tile_bytes = (int64_t)PF_BN * p.k_ss * 2, v_tile_bytes = (int64_t)PF_BN * p.v_ss * 2;
    auto issue_k = [&](int t, char* dst) __attribute__((always_inline)) {
        int64_t rem = (int64_t)(Skv - t * PF_BN - 1) * p.k_ss * 2 + D * 2;    // bytes to the end of the last valid row
        if (rem > 0x7fffffffLL) rem = 0x7fffffffLL;
        __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)kp + t * k_tile_bytes), 0, (int)rem, 0x00020000);
#pragma unroll
        for (int c = 0; c < LPW; ++c)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void*)(dst + (wave * LPW + c) * 1024), 16, k_voff[c], 0, 0, 0);
    };
    auto issue_v = [&](int t, char* dst) __attribute__((always_inline)) {
        int64_t rem = (int64_t)(Skv - t * PF_BN - 1) * p.v_ss * 2 + D * 2;
        if (rem > 0x7fffffffLL) rem = 0x7fffffffLL;
        __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)vp + t * v_tile_bytes), 0, (int)rem, 0x00020000);
#pragma unroll
        for (int c = 0; c < LPW; ++c)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void*)(dst + (wave * LPW + c) * 1024), 16, v_voff[c], 0, 0, 0);
    };

    // ---- LDS read addresses (byte offsets inside a tile) ---------------------------------------
    // K operand: lane (ql, g) reads row 32*half + ql, logical chunk 2*s + g, stored at slot
    // (2*s + g) ^ fk(ql): address = k_base ^ (s << 5) + half * 32 rows.
    const int k_base = ql * L::ROWB + ((g ^ L::fk(ql)) << 4);
    // V operand (transposing read): the 16 lanes of a group fetch a 4-key x 16-d patch (lane n: key
    // n/4, d 4*(n%4)..+3) and receive (d = n, keys 0..3).  Row 32*half + 16*ks + 8*h + 4*g + n/4,
    // logical chunk 4*db + 2*dh + (n%4)/2, stored at slot chunk ^ fv(row):
    // address = v_base ^ (db << 6) + row terms.
    int v_base;
    {
        const int n = lane & 15, dh = (lane >> 4) & 1;
        const int r = 4 * g + (n >> 2);
        const int chunk0 = 2 * dh + ((n & 3) >> 1);
        v_base = r * L::ROWB + ((chunk0 ^ L::fv(r)) << 4) + (n & 1) * 8;
    }

    // ---- Q^T operand, resident in registers ---------------------------------------
    vec8 qreg[NQ];
    {
        const int qi = min(my_i, Sq - 1);
        const T* qrow = qp + (int64_t)qi * p.q_ss + g * 8;
#pragma unroll
        for (int s = 0; s < NQ; ++s) qreg[s] = *(const vec8*)(qrow + s * 16);
    }

    floatx16 o_acc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[db][r] = 0.0f;
    floatx16 s_buf[2];            // S^T of the half-tiles in flight, by half-tile parity
    vec8 p_buf[2][2];             // P^T (storage precision) by half-tile parity, two k-steps of 16 keys
#pragma unroll
    for (int a = 0; a < 2; ++a) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s_buf[a][r] = 0.0f;
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int e = 0; e < 8; ++e) p_buf[a][c][e] = (T)0.0f;
    }
    float m_run = -INFINITY;      // reference maximum of the scaled scores (log2 units); may lag the true maximum
    float l_run = 0.0f;           // this lane's share of the running denominator
    float alpha_pend = 1.0f;      // factor O still has to be multiplied by (after the product in flight)
    bool pend_any = false;        // wavefront-uniform: some lane has alpha_pend != 1
    const float c2 = p.scale * 1.4426950408889634f;

    // ---- one half-iteration ------------------------------------------------------------------------
    // XP      parity of the half-tile x whose scores the matrix pipe produces (s_buf[XP]); the vector ALU
    //         turns s_buf[1-XP] into p_buf[1-XP]; the matrix pipe then consumes p_buf[XP] (half-tile x-2).
    // DO_QK / DO_PV / DO_SM switch the three pieces off at the ends of the key range; MASK adds the
    // key-limit test on the produced scores (tiles that cross a causal or length limit).
    auto half_iter = [&](auto XP_, auto DO_QK_, auto DO_PV_, auto DO_SM_, auto MASK_,
                         const char* kbase, const char* vbase, int j0x) __attribute__((always_inline)) {
        constexpr int XP = decltype(XP_)::value, ZP = 1 - XP;
        constexpr bool DO_QK = decltype(DO_QK_)::value != 0, DO_PV = decltype(DO_PV_)::value != 0;
        constexpr bool DO_SM = decltype(DO_SM_)::value != 0, MASK = decltype(MASK_)::value != 0;
        vec8 opb[3];                                   // matrix operands in flight (rotating)
        const float m_use = (m_run == -INFINITY) ? 0.0f : m_run;
        float rsum = 0.0f;

        auto fetch = [&](int f) __attribute__((always_inline)) {
            if (f < NQ) {
                if (DO_QK) opb[f % 3] = *(const vec8*)(kbase + (k_base ^ (f << 5)));
            } else if (DO_PV) {
                const int ks = (f - NQ) / NDB, db = (f - NQ) % NDB;
                const char* a = vbase + (v_base ^ (db << 6)) + ks * 16 * L::ROWB;
                short8v av;
                av.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4v __attribute__((address_space(3)))*)(a));
                av.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4v __attribute__((address_space(3)))*)(a + 8 * L::ROWB));
                opb[f % 3] = __builtin_bit_cast(vec8, av);
            }
        };
        auto mma = [&](int f) __attribute__((always_inline)) {
            if (f < NQ) {
                if (DO_QK) s_buf[XP] = Mma<T>::run(opb[f % 3], qreg[f], s_buf[XP]);
            } else if (DO_PV) {
                const int ks = (f - NQ) / NDB, db = (f - NQ) % NDB;
                o_acc[db] = Mma<T>::run(opb[f % 3], p_buf[XP][ks], o_acc[db]);
            }
        };
        // probabilities of score registers 2*i, 2*i+1 of half-tile z: key 8*(r/4) + 4*g + (r%4) of the half-tile,
        // k-step r/8, element r%8
        auto sm_pair = [&](int i) __attribute__((always_inline)) {
            if (DO_SM) {
                const int r = 2 * i;
                const T e0 = (T)__builtin_amdgcn_exp2f(fmaf(s_buf[ZP][r], c2, -m_use));
                const T e1 = (T)__builtin_amdgcn_exp2f(fmaf(s_buf[ZP][r + 1], c2, -m_use));
                p_buf[ZP][r / 8][r % 8] = e0;
                p_buf[ZP][r / 8][r % 8 + 1] = e1;
                typename Mma<T>::vec2 pr = {e0, e1};
                rsum = Mma<T>::add2(pr, rsum);         // denominator from the rounded probabilities
            }
        };

        if (DO_QK) {
#pragma unroll
            for (int r = 0; r < 16; ++r) s_buf[XP][r] = 0.0f;
        }
        // program order = intended order: operand reads run two slots ahead of the MFMA that uses them,
        // one probability pair rides under each S^T MFMA, the maximum of the new scores under the O^T MFMAs
        fetch(0);
        fetch(1);
        fetch(2);
        float tmax = -INFINITY;
#pragma unroll
        for (int f = 0; f < NSLOT; ++f) {
            mma(f);
            if (f >= 1 && f + 2 < NSLOT) fetch(f + 2);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (i * NQ / 8 == f) sm_pair(i);
            if (DO_QK && f == (NQ + 2 < NSLOT - 2 ? NQ + 2 : NSLOT - 2)) {
                // S^T(x) is complete: key-limit mask (tiles that cross a limit only), then its maximum
                if (MASK) {
                    const int rel = lim_lane - (j0x + 4 * g);      // register r is key j0x + 8*(r/4) + 4*g + (r%4)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        if (8 * (r / 4) + (r % 4) >= rel) s_buf[XP][r] = -INFINITY;
                }
                tmax = s_buf[XP][0];
#pragma unroll
                for (int r = 1; r < 16; ++r) tmax = fmaxf(tmax, s_buf[XP][r]);
            }
        }
        if (DO_QK && DO_PV && DO_SM && !MASK) {
            // Pin that interleaving for the steady-state half-iteration (the instruction scheduler would
            // otherwise cluster the vector work ahead of the MFMAs): per slot one MFMA, the operand reads
            // for two slots later, and the slot's share of vector / transcendental instructions.
            constexpr int DSR = 0x100, MFMA = 0x008, VEC = 0x002 | 0x400;
            __builtin_amdgcn_sched_group_barrier(DSR, 3, 0);
#pragma unroll
            for (int f = 0; f < NSLOT; ++f) {
                __builtin_amdgcn_sched_group_barrier(MFMA, 1, 0);
                if (f >= 1 && f + 2 < NSLOT) {
                    if (f + 2 < NQ) __builtin_amdgcn_sched_group_barrier(DSR, 1, 0);
                    else __builtin_amdgcn_sched_group_barrier(DSR, 2, 0);
                }
                if (f < NQ) __builtin_amdgcn_sched_group_barrier(VEC, 6 * (8 / NQ), 0);
                else if (f >= NQ + 2) __builtin_amdgcn_sched_group_barrier(VEC, 2, 0);
            }
        }
        if (DO_SM) l_run += rsum;
        // ---- boundary: O catches up with the previous raise of m; then decide about this one ----
        if (pend_any) {
            asm volatile("" ::);           // keeps this rare path a branch (otherwise it is flattened into 16*NDB multiplies by 1)
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) o_acc[db][r] *= alpha_pend;
        }
        if (DO_QK) {
            tmax = xor32_max(tmax) * c2;
            const bool need = tmax > m_run + PF_RESCALE_THRESHOLD;
            const float m_new = need ? fmaxf(m_run, tmax) : m_run;
            alpha_pend = __builtin_amdgcn_exp2f(m_run - ((m_new == -INFINITY) ? 0.0f : m_new));   // 1 when m stays
            alpha_pend = need ? alpha_pend : 1.0f;
            l_run *= alpha_pend;
            m_run = m_new;
            pend_any = __builtin_amdgcn_ballot_w64(need) != 0;
        } else {
            alpha_pend = 1.0f;
            pend_any = false;
        }
    };

    // ---- tile steps -----------------------------------------------------------------------------------
    // step t (0..N): barrier publishes K(t) and V(t-1); loads of K(t+1), V(t) start; half-iterations
    // 2t-1 and 2t run; the wavefront waits for its own loads.
    //   half-iteration 2t-1: S(2t)   from K(t) rows 0..31,  O += P(2t-2) V(t-1) rows 0..31,  P(2t-1)
    //   half-iteration 2t  : S(2t+1) from K(t) rows 32..63, O += P(2t-1) V(t-1) rows 32..63, P(2t)
    auto tile_step = [&](int t, auto PAR_, auto KIND_, auto MASK_) __attribute__((always_inline)) {
        constexpr int par = decltype(PAR_)::value;           // t % 2
        constexpr int KIND = decltype(KIND_)::value;         // 0 first (t = 0), 1 steady, 2 last (t = N)
        char* k_cur = smem + par * TILE;                     // K(t)
        char* k_next = smem + (1 - par) * TILE;              // K(t+1)
        char* v_prev = smem + 2 * TILE + (1 - par) * TILE;   // V(t-1)
        char* v_cur = smem + 2 * TILE + par * TILE;          // V(t)
        __syncthreads();
        if (KIND != 2) {
            if (t + 1 < N) issue_k(t + 1, k_next);
            issue_v(t, v_cur);
        }
        half_iter(ic<0>{}, ic<KIND != 2>{}, ic<KIND != 0>{}, ic<KIND != 0>{}, MASK_, k_cur, v_prev, t * PF_BN);
        half_iter(ic<1>{}, ic<KIND != 2>{}, ic<KIND != 0>{}, ic<KIND != 2>{}, MASK_, k_cur + HALF, v_prev + HALF, t * PF_BN + 32);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };

    if (N > 0) {
        issue_k(0, smem);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        tile_step(0, ic<0>{}, ic<0>{}, ic<1>{});
        // tiles before this one lie entirely below every limit of this wavefront: no mask code
        const int t_mask = lim_wave_min / PF_BN;
        int t = 1;
        for (; t + 1 < N; t += 2) {
            if (t + 1 < t_mask) {
                tile_step(t, ic<1>{}, ic<1>{}, ic<0>{});
                tile_step(t + 1, ic<0>{}, ic<1>{}, ic<0>{});
            } else {
                tile_step(t, ic<1>{}, ic<1>{}, ic<1>{});
                tile_step(t + 1, ic<0>{}, ic<1>{}, ic<1>{});
            }
        }
        if (t < N) {                     // one steady step left (t odd)
            tile_step(t, ic<1>{}, ic<1>{}, ic<1>{});
            ++t;
        }
        if (N & 1) tile_step(N, ic<1>{}, ic<2>{}, ic<0>{});
        else tile_step(N, ic<0>{}, ic<2>{}, ic<0>{});
        if (pend_any) {
            asm volatile("" ::);
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) o_acc[db][r] *= alpha_pend;
        }
    }

    // ---- normalise and store ------------------------------------------------------------------
    const float l_tot = xor32_sum(l_run);
    const float inv = (l_tot == 0.0f) ? __builtin_nanf("") : 1.0f / l_tot;   // no visible key: NaN, as the reference
    if (my_i < Sq) {
        T* orow = op + (int64_t)my_i * p.o_ss;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                typedef T vec4 __attribute__((ext_vector_type(4)));
                vec4 w;
#pragma unroll
                for (int e = 0; e < 4; ++e) w[e] = (T)(o_acc[db][r4 * 4 + e] * inv);
                *(vec4*)(orow + db * 32 + r4 * 8 + g * 4) = w;
            }
    }
#endif
}

template <typename T, int D>
static hipError_t launch_pipe_t(const SdpaParams& p, hipStream_t stream)
{
    const int nqb = (p.Sq + PF_BM - 1) / PF_BM;
    const int64_t total = (int64_t)nqb * p.Hq * p.B;
    hipLaunchKernelGGL((sdpa_prefill_pipe_kernel<T, D>), dim3((unsigned)total), dim3(256), 0, stream, p);
    return hipGetLastError();
}

// Same preconditions as launch_sdpa_prefill_mfma.
hipError_t launch_sdpa_prefill_pipe(const SdpaParams& p, int dtype, hipStream_t stream)
{
    if (dtype == 1) return p.D == 128 ? launch_pipe_t<f16_t, 128>(p, stream) : launch_pipe_t<f16_t, 64>(p, stream);
    return p.D == 128 ? launch_pipe_t<bf16_t, 128>(p, stream) : launch_pipe_t<bf16_t, 64>(p, stream);
}

}  // namespace incin_rocm
