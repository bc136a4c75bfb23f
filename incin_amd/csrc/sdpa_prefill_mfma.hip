// bf16 / f16 attention forward on the gfx950 matrix cores (prefill shapes).
//
// Computes the function of the reference CPU composition
// (crates/incin-backends/src/cpu/ops/shape_ops.rs:1245-1269) for D == Dv in
// {64, 128}, optional causal mask and per-batch key lengths, MHA and GQA, with
// f32 accumulation and an online softmax: no score tensor is ever materialised.
//
// Shape of the computation (one workgroup = 4 wavefronts = 128 query rows, one
// wavefront = 32 query rows, key tile = 64 keys):
//
//   S^T = K_tile Q^T     v_mfma_f32_32x32x16: A = K rows from LDS (16-byte reads),
//                        B = Q^T held in registers for the whole kernel.
//                        In the 32x32 result a lane owns ONE query (column
//                        lane%32) and 16 keys per 32-key block, so the row max
//                        and row sum of the softmax are in-lane reductions plus
//                        a single exchange with lane^32.
//   P^T                  exp2 of the scaled scores, rounded to the storage type
//                        in registers; the accumulator layout of S^T is already
//                        the B-operand layout of the next product (the key
//                        order inside a k-step is a fixed permutation, which
//                        the V reads below follow).
//   O^T += V^T P^T       A = V^T read from the row-major V tile in LDS with the
//                        transposing LDS read (ds_read_b64_tr_b16).
//
// K and V tiles are fetched from global memory into registers one tile ahead
// and stored to padded LDS rows (K: +16 B, V: +64 B per row, chosen so the two
// read patterns above are bank-conflict free).
#include "sdpa_params.h"

namespace incin_rocm {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));
typedef bf16_t bf16x8 __attribute__((ext_vector_type(8)));
typedef f16_t f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
typedef unsigned int uint2v __attribute__((ext_vector_type(2)));

template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
    typedef bf16x8 vec8;
    static __device__ __forceinline__ floatx16 run(vec8 a, vec8 b, floatx16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Mma<f16_t> {
    typedef f16x8 vec8;
    static __device__ __forceinline__ floatx16 run(vec8 a, vec8 b, floatx16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

constexpr int PF_BM = 128;     // query rows per workgroup
constexpr int PF_BN = 64;      // keys per tile
constexpr int PF_WAVES = 4;

template <int D> struct PfLayout {
    static constexpr int KSTR = D + 8;     // elements per K row in LDS (+16 B)
    static constexpr int VSTR = D + 32;    // elements per V row in LDS (+64 B)
    static constexpr int K_ELEMS = PF_BN * KSTR;
    static constexpr int V_ELEMS = PF_BN * VSTR;
    static constexpr int LDS_BYTES = (K_ELEMS + V_ELEMS) * 2;
};

template <typename T, int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void sdpa_prefill_mfma_kernel(SdpaParams p)
{
    typedef typename Mma<T>::vec8 vec8;
    typedef PfLayout<D> L;
    constexpr int NSTEP = D / 16;          // k-steps of the S^T product
    constexpr int NDB = D / 32;            // 32-wide blocks of the head dimension
    constexpr int CHUNKS = PF_BN * D / 8;  // 16-byte chunks per tile
    constexpr int CPT = CHUNKS / 256;      // chunks per thread
    constexpr int CPR = D / 8;             // chunks per row

    __shared__ __attribute__((aligned(16))) T Ks[L::K_ELEMS];
    __shared__ __attribute__((aligned(16))) T Vs[L::V_ELEMS];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
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
    // keys visible to this workgroup / this wavefront / this lane's query
    int j_end = kv_len;
    const int my_i = q0 + wave * 32 + ql;
    int lim_lane = kv_len, lim_wave_min = kv_len, lim_wave_max = kv_len;
    if (p.causal) {
        const int last_row = min(q0 + PF_BM - 1, Sq - 1);
        j_end = clampi(last_row + coff + 1, 0, kv_len);
        lim_lane = clampi(my_i + coff + 1, 0, kv_len);
        lim_wave_min = clampi(q0 + wave * 32 + coff + 1, 0, kv_len);
        lim_wave_max = clampi(min(q0 + wave * 32 + 31, Sq - 1) + coff + 1, 0, kv_len);
    }
    const int n_tiles = (j_end + PF_BN - 1) / PF_BN;

    // ---- Q^T operand, resident in registers ---------------------------------------
    vec8 qreg[NSTEP];
    {
        const int qi = min(my_i, Sq - 1);
        const T* qrow = qp + (int64_t)qi * p.q_ss + g * 8;
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) qreg[s] = *(const vec8*)(qrow + s * 16);
    }

    floatx16 o_acc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[db][r] = 0.0f;
    float m_run = -INFINITY;      // running max of the scaled scores, log2 units
    float l_run = 0.0f;           // this lane's share of the running denominator
    const float c2 = p.scale * 1.4426950408889634f;

    // ---- tile prefetch registers -----------------------------------------------------
    uint4v kpre[CPT], vpre[CPT];
    auto fetch = [&](int j0) {
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            const int chunk = tid + c * 256;
            const int row = chunk / CPR, col = (chunk % CPR) * 8;
            const int j = min(j0 + row, Skv - 1);
            kpre[c] = *(const uint4v*)(kp + (int64_t)j * p.k_ss + col);
            vpre[c] = *(const uint4v*)(vp + (int64_t)j * p.v_ss + col);
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int c = 0; c < CPT; ++c) {
            const int chunk = tid + c * 256;
            const int row = chunk / CPR, col = (chunk % CPR) * 8;
            *(uint4v*)(Ks + row * L::KSTR + col) = kpre[c];
            *(uint4v*)(Vs + row * L::VSTR + col) = vpre[c];
        }
    };

    if (n_tiles > 0) fetch(0);

    for (int t = 0; t < n_tiles; ++t) {
        const int j0 = t * PF_BN;
        __syncthreads();                       // every wavefront has finished reading the previous tile
        stash();
        __syncthreads();
        if (t + 1 < n_tiles) fetch(j0 + PF_BN);

        if (j0 >= lim_wave_max) continue;      // no query of this wavefront sees this tile (uniform per wavefront)

        // ---- S^T = K Q^T ----------------------------------------------------------
        floatx16 s_acc[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) s_acc[kb][r] = 0.0f;
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const vec8 a = *(const vec8*)(Ks + (kb * 32 + ql) * L::KSTR + s * 16 + g * 8);
                s_acc[kb] = Mma<T>::run(a, qreg[s], s_acc[kb]);
            }
        }

        // ---- masking (only tiles that cross a limit) --------------------------------
        // register r of block kb is key j0 + 32*kb + 8*(r/4) + 4*g + (r%4)
        if (j0 + PF_BN > lim_wave_min) {
            const int rel = lim_lane - (j0 + 4 * g);
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int kofs = 32 * kb + 8 * (r / 4) + (r % 4);
                    if (kofs >= rel) s_acc[kb][r] = -INFINITY;
                }
        }

        // ---- online softmax --------------------------------------------------------------
        float tmax = s_acc[0][0];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, s_acc[kb][r]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m_run, tmax * c2);
        const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
        m_run = m_new;
        float rsum = 0.0f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float e = __builtin_amdgcn_exp2f(fmaf(s_acc[kb][r], c2, -m_use));
                s_acc[kb][r] = e;
                rsum += e;
            }
        l_run = fmaf(l_run, alpha, rsum);
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) o_acc[db][r] *= alpha;

        // ---- O^T += V^T P^T ---------------------------------------------------------------
        // k-step ks covers registers 8*(ks%2)..+7 of key block ks/2; element e of
        // a lane is key 32*(ks/2) + 16*(ks%2) + 8*(e/4) + 4*g + (e%4).
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            vec8 pb;
#pragma unroll
            for (int e = 0; e < 8; ++e) pb[e] = (T)s_acc[ks / 2][8 * (ks % 2) + e];
            const int kbase = 32 * (ks / 2) + 16 * (ks % 2) + 4 * g;
            // transposing read: the 16 lanes of a group fetch a 4-key x 16-d patch
            // (lane n: key n/4, d 4*(n%4)..+3) and receive (d = n, keys 0..3).
            const int n = lane & 15, dh = (lane >> 4) & 1;
#pragma unroll
            for (int db = 0; db < NDB; ++db) {
                const T* base = Vs + (kbase + (n >> 2)) * L::VSTR + db * 32 + dh * 16 + (n & 3) * 4;
                const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (short4v __attribute__((address_space(3)))*)(base));
                const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (short4v __attribute__((address_space(3)))*)(base + 8 * L::VSTR));
                short8v av;
                av.lo = lo;
                av.hi = hi;
                o_acc[db] = Mma<T>::run(__builtin_bit_cast(vec8, av), pb, o_acc[db]);
            }
        }
    }

    // ---- normalise and store ------------------------------------------------------------------
    const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
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
}

template <typename T, int D>
static hipError_t launch_prefill_t(const SdpaParams& p, hipStream_t stream)
{
    const int nqb = (p.Sq + PF_BM - 1) / PF_BM;
    const int64_t total = (int64_t)nqb * p.Hq * p.B;
    hipLaunchKernelGGL((sdpa_prefill_mfma_kernel<T, D>), dim3((unsigned)total), dim3(256), 0, stream, p);
    return hipGetLastError();
}

// Host has validated: dtype f16/bf16, D == Dv in {64,128}, scale > 0, no dense
// mask, rows 16-byte aligned with unit last-dim stride.
hipError_t launch_sdpa_prefill_mfma(const SdpaParams& p, int dtype, hipStream_t stream)
{
    if (dtype == 1) return p.D == 128 ? launch_prefill_t<f16_t, 128>(p, stream) : launch_prefill_t<f16_t, 64>(p, stream);
    return p.D == 128 ? launch_prefill_t<bf16_t, 128>(p, stream) : launch_prefill_t<bf16_t, 64>(p, stream);
}

}  // namespace incin_rocm
