// Generic attention forward: fp32 FMA arithmetic, any of f32/f16/bf16 storage,
// D and Dv up to DMAX, dense additive mask + causal + per-batch key lengths.
//
// This is the kernel every request can fall back on; the MFMA and split-KV
// kernels cover the shapes that matter for throughput.  It computes the same
// function as the reference CPU composition
// (crates/incin-backends/src/cpu/ops/shape_ops.rs:1245-1269) with an online
// softmax instead of materialised score tensors.
//
// Tiling: one workgroup (256 threads = 16 x 16) owns 64 query rows; it walks
// the keys 64 at a time.  Thread (ty, tx) owns rows 4*ty..4*ty+3 and key
// columns tx, tx+16, tx+32, tx+48 of the score tile, and the same rows times
// output columns tx + 16*c of the accumulator.  Q, the current K (then V) tile
// and the probability tile live in LDS as f32 with one float of row padding,
// which makes every LDS access of the two inner loops conflict-free.
#include <atomic>

#include "sdpa_params.h"

namespace incin_rocm {

constexpr int GEN_BM = 64;
constexpr int GEN_BN = 64;

template <typename T, int DMAX>
__global__ __launch_bounds__(256) void sdpa_generic_kernel(SdpaParams p)
{
    constexpr int DP = DMAX + 1;
    constexpr int PP = GEN_BN + 1;
    constexpr int NC = DMAX / 16;
    extern __shared__ float smem[];
    float* Qs = smem;                    // [GEN_BM][DP]
    float* KVs = Qs + GEN_BM * DP;       // [GEN_BN][DP]
    float* Ps = KVs + GEN_BN * DP;       // [GEN_BM][PP]

    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int q0 = blockIdx.x * GEN_BM, hq = blockIdx.y, b = blockIdx.z;
    const int hkv = hq / p.G;
    const int D = p.D, Dv = p.Dv, Sq = p.Sq, Skv = p.Skv;
    const T* qp = (const T*)p.q + (int64_t)b * p.q_sb + (int64_t)hq * p.q_sh;
    const T* kp = (const T*)p.k + (int64_t)b * p.k_sb + (int64_t)hkv * p.k_sh;
    const T* vp = (const T*)p.v + (int64_t)b * p.v_sb + (int64_t)hkv * p.v_sh;
    T* op = (T*)p.o + (int64_t)b * p.o_sb + (int64_t)hq * p.o_sh;
    const T* mp = p.mask ? (const T*)p.mask + (int64_t)b * p.m_sb + (int64_t)hq * p.m_sh : nullptr;

    for (int idx = tid; idx < GEN_BM * D; idx += 256) {
        int r = idx / D, d = idx - r * D;
        int row = q0 + r;
        Qs[r * DP + d] = row < Sq ? to_f32(qp[(int64_t)row * p.q_ss + d]) : 0.0f;
    }

    int kv_len = Skv;
    if (p.kv_lens) kv_len = clampi(p.kv_lens[b], 0, Skv);
    int j_end = kv_len;                                     // keys >= j_end are masked for every row of this block
    if (p.causal) {
        int last_row = (q0 + GEN_BM - 1 < Sq - 1) ? q0 + GEN_BM - 1 : Sq - 1;
        int lim = causal_limit(last_row, Sq, Skv);
        if (lim < j_end) j_end = lim;
        if (j_end < 0) j_end = 0;
    }

    float m_run[4], l_run[4], acc[4][NC];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        m_run[r] = -INFINITY;
        l_run[r] = 0.0f;
#pragma unroll
        for (int c = 0; c < NC; ++c) acc[r][c] = 0.0f;
    }

    for (int j0 = 0; j0 < j_end; j0 += GEN_BN) {
        __syncthreads();                                    // previous tile's V and P fully consumed (and Q stored)
        for (int idx = tid; idx < GEN_BN * D; idx += 256) {
            int r = idx / D, d = idx - r * D;
            int j = j0 + r;
            KVs[r * DP + d] = j < kv_len ? to_f32(kp[(int64_t)j * p.k_ss + d]) : 0.0f;     // rows past the key count are never read
        }
        __syncthreads();

        float s[4][4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int c = 0; c < 4; ++c) s[r][c] = 0.0f;
        for (int d = 0; d < D; ++d) {
            float qv[4], kv[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) qv[r] = Qs[(ty * 4 + r) * DP + d];
#pragma unroll
            for (int c = 0; c < 4; ++c) kv[c] = KVs[(tx + 16 * c) * DP + d];
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int c = 0; c < 4; ++c) s[r][c] = fmaf(qv[r], kv[c], s[r][c]);
        }

#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int i = q0 + ty * 4 + r;
            const int lim = p.causal ? causal_limit(i, Sq, Skv) : Skv;
            float tmax = -INFINITY;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int j = j0 + tx + 16 * c;
                float x = s[r][c] * p.scale;
                if (mp && i < Sq && j < Skv) x += to_f32(mp[(int64_t)i * p.m_si + (int64_t)j * p.m_sj]);
                if (j >= kv_len || j >= lim) x = -INFINITY;
                s[r][c] = x;
                tmax = fmaxf(tmax, x);
            }
#pragma unroll
            for (int off = 8; off >= 1; off >>= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, off, 16));
            const float m_new = fmaxf(m_run[r], tmax);
            const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
            const float alpha = expf(m_run[r] - m_use);
            float rsum = 0.0f;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                float e = expf(s[r][c] - m_use);
                rsum += e;
                Ps[(ty * 4 + r) * PP + tx + 16 * c] = e;
            }
#pragma unroll
            for (int off = 8; off >= 1; off >>= 1) rsum += __shfl_xor(rsum, off, 16);
            l_run[r] = l_run[r] * alpha + rsum;
            m_run[r] = m_new;
#pragma unroll
            for (int c = 0; c < NC; ++c) acc[r][c] *= alpha;
        }
        __syncthreads();                                    // K tile consumed, P tile complete
        for (int idx = tid; idx < GEN_BN * Dv; idx += 256) {
            int r = idx / Dv, d = idx - r * Dv;
            int j = j0 + r;
            KVs[r * DP + d] = j < kv_len ? to_f32(vp[(int64_t)j * p.v_ss + d]) : 0.0f;
        }
        __syncthreads();
        for (int jj = 0; jj < GEN_BN; ++jj) {
            float pv[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) pv[r] = Ps[(ty * 4 + r) * PP + jj];
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                if (tx + 16 * c < Dv) {
                    float vv = KVs[jj * DP + tx + 16 * c];
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[r][c] = fmaf(pv[r], vv, acc[r][c]);
                }
            }
        }
    }

#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int i = q0 + ty * 4 + r;
        if (i >= Sq) continue;
        const float inv = 1.0f / l_run[r];                  // l == 0 (no visible key): 0 * inf = NaN, as the reference
        if (p.lse && tx == 0)
            p.lse[((int64_t)b * p.Hq + hq) * Sq + i] = l_run[r] == 0.0f ? -INFINITY : m_run[r] + logf(l_run[r]);
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int col = tx + 16 * c;
            if (col < Dv) {
                float val = (l_run[r] == 0.0f) ? __builtin_nanf("") : acc[r][c] * inv;
                if (Skv == 0) val = 0.0f;                   // empty key axis: the reference's second matmul leaves zeros
                op[(int64_t)i * p.o_ss + col] = from_f32<T>(val);
            }
        }
    }
}

template <typename T, int DMAX>
static hipError_t launch_generic_t(const SdpaParams& p, hipStream_t stream)
{
    size_t lds = (size_t)(GEN_BM * (DMAX + 1) + GEN_BN * (DMAX + 1) + GEN_BM * (GEN_BN + 1)) * sizeof(float);
    auto kern = sdpa_generic_kernel<T, DMAX>;
    hipError_t e;
    // the dynamic-LDS limit of this instance is raised once per device, not per launch
    static std::atomic<uint64_t> prepared{0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    const uint64_t bit = 1ull << (dev & 63);
    if (!(prepared.load(std::memory_order_acquire) & bit)) {
        e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        prepared.fetch_or(bit, std::memory_order_release);
    }
    dim3 grid((p.Sq + GEN_BM - 1) / GEN_BM, p.Hq, p.B);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, p);
    return hipGetLastError();
}

template <typename T>
static hipError_t launch_generic_d(const SdpaParams& p, hipStream_t stream)
{
    int dm = p.D > p.Dv ? p.D : p.Dv;
    if (dm <= 64) return launch_generic_t<T, 64>(p, stream);
    if (dm <= 128) return launch_generic_t<T, 128>(p, stream);
    return launch_generic_t<T, 256>(p, stream);
}

// dtype: 0 f32, 1 f16, 2 bf16.  Host has validated max(D, Dv) <= 256.
hipError_t launch_sdpa_generic(const SdpaParams& p, int dtype, hipStream_t stream)
{
    switch (dtype) {
        case 0: return launch_generic_d<float>(p, stream);
        case 1: return launch_generic_d<f16_t>(p, stream);
        default: return launch_generic_d<bf16_t>(p, stream);
    }
}

}  // namespace incin_rocm
