// Split-KV attention for a handful of query rows over a long key/value cache
// (single-token decode, MHA and GQA), plus the kernel that combines the
// per-split partial softmax results.
//
// The work is bandwidth-bound: every K and V element is read exactly once,
// with 16-byte loads that cover whole rows contiguously, and no LDS staging of
// K or V.  A workgroup (4 wavefronts) owns one (batch, kv-head, split) and up
// to RMAX query rows that share that kv-head (the G query heads of a GQA group
// times Sq), so K/V are read once per group.  Inside a wavefront LPR = D/VEC
// lanes cooperate on one key row; the 64/LPR such lane groups each keep their
// own running (max, sum, accumulator) stream, merged once through LDS when the
// split is done.
//
// Partial results: ws_acc[b,hq,i,split,:] = sum_j exp(s_j - m) v_j,
// ws_ml[b,hq,i,split] = (m, sum_j exp(s_j - m)); the combine kernel rescales
// them to a common max.  With num_splits == 1 the first kernel writes the
// final output itself.
#include <atomic>

#include "sdpa_params.h"

namespace incin_rocm {

template <typename T> struct Vec16;
template <> struct Vec16<float> { typedef float type __attribute__((ext_vector_type(4))); static constexpr int N = 4; };
template <> struct Vec16<f16_t> { typedef f16_t type __attribute__((ext_vector_type(8))); static constexpr int N = 8; };
template <> struct Vec16<bf16_t> { typedef bf16_t type __attribute__((ext_vector_type(8))); static constexpr int N = 8; };

// exp(x): full-precision library routine for f32 storage (1e-5 tolerance),
// hardware exp2 on a pre-scaled argument for 16-bit storage.
template <typename T> struct Softexp {
    static constexpr float kPre = 1.4426950408889634f;       // scores are kept in log2 units
    static __device__ __forceinline__ float ex(float x) { return __builtin_amdgcn_exp2f(x); }
};
template <> struct Softexp<float> {
    static constexpr float kPre = 1.0f;
    static __device__ __forceinline__ float ex(float x) { return expf(x); }
};

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float x)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}

// Sum over each aligned group of LPR consecutive lanes; every lane of the
// group ends up with the total.
template <int LPR>
__device__ __forceinline__ float group_sum(float x)
{
    if (LPR >= 2) x += dpp_f32<0xB1>(x);        // quad_perm [1,0,3,2]
    if (LPR >= 4) x += dpp_f32<0x4E>(x);        // quad_perm [2,3,0,1]
    if (LPR >= 8) x += dpp_f32<0x141>(x);       // row_half_mirror
    if (LPR >= 16) x += dpp_f32<0x140>(x);      // row_mirror
    if (LPR >= 32) x += __shfl_xor(x, 16, 64);
    if (LPR >= 64) x += __shfl_xor(x, 32, 64);
    return x;
}

// DENSE: a dense additive mask (any broadcast strides): its value for (row, key) is added to the scaled score - what an
// additive position bias or a mask tensor with holes needs at decode time.
template <typename T, int D, int RMAX, int U, bool DENSE = false>
__global__ __launch_bounds__(256) void sdpa_decode_split_kernel(SdpaParams p)
{
    typedef typename Vec16<T>::type vec_t;
    constexpr int VEC = Vec16<T>::N;
    constexpr int LPR = D / VEC;          // lanes per key row
    constexpr int KPL = 64 / LPR;         // key rows per wavefront-wide load
    constexpr int KT = U * KPL;           // keys per wavefront tile
    constexpr int NSTREAM = 4 * KPL;
    static_assert(LPR >= 1 && LPR <= 64 && (64 % LPR) == 0, "row must fit a wavefront");

    extern __shared__ float smem[];
    float* s_acc = smem;                                   // [NSTREAM][RMAX][D]
    float* s_ml = smem + NSTREAM * RMAX * D;               // [NSTREAM][RMAX][2]

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane / LPR;
    const int dl = (lane % LPR) * VEC;
    const int R = p.G * p.Sq;
    const int nchunks = (R + RMAX - 1) / RMAX;
    const int split = blockIdx.x;
    const int hkv = blockIdx.y / nchunks, r0 = (blockIdx.y % nchunks) * RMAX;
    const int b = blockIdx.z;
    const int Skv = p.Skv, Sq = p.Sq;

    int kv_len = Skv;
    if (p.kv_lens) kv_len = clampi(p.kv_lens[b], 0, Skv);
    const int k_begin = split * p.split_len;
    int k_end = k_begin + p.split_len;
    if (k_end > kv_len) k_end = kv_len;

    const float sc = p.scale * Softexp<T>::kPre;
    float qf[RMAX][VEC];
    int lim[RMAX];
    [[maybe_unused]] const T* mrow[RMAX];      // this row of the dense mask
#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
        const int row = r0 + r;
        const bool valid = row < R;
        const int g = valid ? row / Sq : 0, i = valid ? row % Sq : 0;
        const T* qp = (const T*)p.q + (int64_t)b * p.q_sb + (int64_t)(hkv * p.G + g) * p.q_sh + (int64_t)i * p.q_ss + dl;
        vec_t qv = *(const vec_t*)qp;
#pragma unroll
        for (int e = 0; e < VEC; ++e) qf[r][e] = valid ? to_f32(qv[e]) : 0.0f;
        int l = k_end;
        if (p.causal) {
            int cl = causal_limit(i, Sq, Skv);
            if (cl < l) l = cl;
        }
        lim[r] = valid ? l : 0;
        if (DENSE) mrow[r] = (const T*)p.mask + (int64_t)b * p.m_sb + (int64_t)(hkv * p.G + g) * p.m_sh + (int64_t)i * p.m_si;
    }

    float m_run[RMAX], l_run[RMAX], acc[RMAX][VEC];
#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
        m_run[r] = -INFINITY;
        l_run[r] = 0.0f;
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[r][e] = 0.0f;
    }

    const T* kp = (const T*)p.k + (int64_t)b * p.k_sb + (int64_t)hkv * p.k_sh + dl;
    const T* vp = (const T*)p.v + (int64_t)b * p.v_sb + (int64_t)hkv * p.v_sh + dl;

    // Rows at and beyond k_end (the end of the split, at most the batch entry's key count) are never read: a lane whose
    // key lies there re-reads the split's last row, and its score is masked below.  What an unwritten cache tail holds
    // (NaN bit patterns included) therefore cannot reach the result through 0 * v.
    const int k_last = k_end - 1;
    for (int t0 = k_begin + wave * KT; t0 < k_end; t0 += 4 * KT) {
        vec_t kreg[U], vreg[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            int key = t0 + u * KPL + sub;
            if (key > k_last) key = k_last;
            kreg[u] = __builtin_nontemporal_load((const vec_t*)(kp + (int64_t)key * p.k_ss));
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            int key = t0 + u * KPL + sub;
            if (key > k_last) key = k_last;
            vreg[u] = __builtin_nontemporal_load((const vec_t*)(vp + (int64_t)key * p.v_ss));
        }

        float s[RMAX][U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float kf[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) kf[e] = to_f32(kreg[u][e]);
            const int key = t0 + u * KPL + sub;
#pragma unroll
            for (int r = 0; r < RMAX; ++r) {
                float part = 0.0f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) part = fmaf(qf[r][e], kf[e], part);
                part = group_sum<LPR>(part) * sc;
                if (DENSE) part = fmaf(to_f32(mrow[r][(int64_t)min(key, k_last) * p.m_sj]), Softexp<T>::kPre, part);
                s[r][u] = (key < lim[r]) ? part : -INFINITY;
            }
        }
#pragma unroll
        for (int r = 0; r < RMAX; ++r) {
            float tmax = s[r][0];
#pragma unroll
            for (int u = 1; u < U; ++u) tmax = fmaxf(tmax, s[r][u]);
            const float m_new = fmaxf(m_run[r], tmax);
            const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
            const float alpha = Softexp<T>::ex(m_run[r] - m_use);
            m_run[r] = m_new;
            float rs = 0.0f;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                s[r][u] = Softexp<T>::ex(s[r][u] - m_use);
                rs += s[r][u];
            }
            l_run[r] = l_run[r] * alpha + rs;
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[r][e] *= alpha;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float vf[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) vf[e] = to_f32(vreg[u][e]);
#pragma unroll
            for (int r = 0; r < RMAX; ++r)
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[r][e] = fmaf(s[r][u], vf[e], acc[r][e]);
        }
    }

    // merge the NSTREAM streams of this workgroup
    const int stream_id = wave * KPL + sub;
#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) s_acc[(stream_id * RMAX + r) * D + dl + e] = acc[r][e];
        if ((lane % LPR) == 0) {
            s_ml[(stream_id * RMAX + r) * 2 + 0] = m_run[r];
            s_ml[(stream_id * RMAX + r) * 2 + 1] = l_run[r];
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < RMAX * D; idx += 256) {
        const int r = idx / D, d = idx - r * D;
        const int row = r0 + r;
        if (row >= R) continue;
        float M = -INFINITY;
        for (int s2 = 0; s2 < NSTREAM; ++s2) M = fmaxf(M, s_ml[(s2 * RMAX + r) * 2]);
        const float M_use = (M == -INFINITY) ? 0.0f : M;
        float L = 0.0f, A = 0.0f;
        for (int s2 = 0; s2 < NSTREAM; ++s2) {
            const float w = Softexp<T>::ex(s_ml[(s2 * RMAX + r) * 2] - M_use);
            L = fmaf(w, s_ml[(s2 * RMAX + r) * 2 + 1], L);
            A = fmaf(w, s_acc[(s2 * RMAX + r) * D + d], A);
        }
        const int g = row / Sq, i = row % Sq;
        const int hq = hkv * p.G + g;
        if (p.num_splits == 1) {
            T* op = (T*)p.o + (int64_t)b * p.o_sb + (int64_t)hq * p.o_sh + (int64_t)i * p.o_ss;
            op[d] = from_f32<T>(L == 0.0f ? __builtin_nanf("") : A / L);
            if (p.lse && d == 0) p.lse[((int64_t)b * p.Hq + hq) * Sq + i] = L == 0.0f ? -INFINITY : M / Softexp<T>::kPre + logf(L);
        } else {
            const int64_t slot = (((int64_t)b * p.Hq + hq) * Sq + i) * p.num_splits + split;
            p.ws_acc[slot * D + d] = A;
            if (d == 0) {
                p.ws_ml[slot * 2 + 0] = M;
                p.ws_ml[slot * 2 + 1] = L;
            }
        }
    }
}

// One workgroup per (b, hq, i) row: rescale the partials of all splits to their common maximum and normalise.  A
// thread holds 4 consecutive output elements; the D / 4 threads of a group walk the splits group, group + NG, ..., so
// that NG splits are read side by side (a launch with hundreds of splits and few rows would otherwise walk them one
// after the other), and the groups' sums meet in LDS.  blockDim.x = NG * D / 4, a multiple of 64.
template <typename T, int D>
__global__ __launch_bounds__(256) void sdpa_combine_kernel(SdpaParams p)
{
    constexpr int TPR = D / 4;
    constexpr int NG_MAX = 256 / TPR;
    typedef float f4 __attribute__((ext_vector_type(4)));
    __shared__ float s_max[4];
    __shared__ f4 s_acc[NG_MAX][TPR];
    __shared__ float s_l[NG_MAX];
    const int64_t row = blockIdx.x;                    // (b * Hq + hq) * Sq + i
    const int tid = threadIdx.x;
    const int ng = blockDim.x / TPR;
    const int i = (int)(row % p.Sq);
    const int64_t bh = row / p.Sq;
    const int hq = (int)(bh % p.Hq), b = (int)(bh / p.Hq);
    const float* ml = p.ws_ml + row * p.num_splits * 2;
    const float* ac = p.ws_acc + row * p.num_splits * D;
    float m = -INFINITY;
    for (int s = tid; s < p.num_splits; s += blockDim.x) m = fmaxf(m, ml[s * 2]);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if ((tid & 63) == 0) s_max[tid >> 6] = m;
    __syncthreads();
    float M = s_max[0];
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w) M = fmaxf(M, s_max[w]);
    const float M_use = (M == -INFINITY) ? 0.0f : M;
    const int grp = tid / TPR, c = tid % TPR;
    f4 A = {0.0f, 0.0f, 0.0f, 0.0f};
    float L = 0.0f;
    for (int s = grp; s < p.num_splits; s += ng) {
        const float w = Softexp<T>::ex(ml[s * 2] - M_use);
        L = fmaf(w, ml[s * 2 + 1], L);
        const f4 a = *(const f4*)(ac + (int64_t)s * D + 4 * c);
#pragma unroll
        for (int e = 0; e < 4; ++e) A[e] = fmaf(w, a[e], A[e]);
    }
    s_acc[grp][c] = A;
    if (c == 0) s_l[grp] = L;
    __syncthreads();
    if (tid < TPR) {
        for (int g2 = 1; g2 < ng; ++g2) {
            const f4 a = s_acc[g2][tid];
#pragma unroll
            for (int e = 0; e < 4; ++e) A[e] += a[e];
            L += s_l[g2];
        }
        typedef T vec4 __attribute__((ext_vector_type(4)));
        vec4 w;
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = from_f32<T>(L == 0.0f ? __builtin_nanf("") : A[e] / L);
        T* op = (T*)p.o + (int64_t)b * p.o_sb + (int64_t)hq * p.o_sh + (int64_t)i * p.o_ss;
        if (4 * tid < p.Dv) *(vec4*)(op + 4 * tid) = w;      // (the partial rows are as wide as the kernel instance, the output as V's rows)
        // the row's softmax normaliser, natural log (the maxima are in log2 units for 16-bit storage)
        if (p.lse && tid == 0) p.lse[row] = L == 0.0f ? -INFINITY : M / Softexp<T>::kPre + logf(L);
    }
}

template <typename T, int D>
static hipError_t launch_combine_t(const SdpaParams& p, hipStream_t stream)
{
    constexpr int TPR = D / 4;
    int ng = 64 / TPR;                                  // at least one wavefront
    while (ng < 256 / TPR && ng < p.num_splits) ng *= 2;
    hipLaunchKernelGGL((sdpa_combine_kernel<T, D>), dim3((unsigned)((int64_t)p.B * p.Hq * p.Sq)), dim3(ng * TPR), 0, stream, p);
    return hipGetLastError();
}

// The partial results of a split-KV launch (rows of p.Dp floats: 64, 128 or 256) into the output.
hipError_t launch_sdpa_combine(const SdpaParams& p, int dtype, hipStream_t stream)
{
    if (p.Dp == 256) return dtype == 0 ? launch_combine_t<float, 256>(p, stream) : dtype == 1 ? launch_combine_t<f16_t, 256>(p, stream) : launch_combine_t<bf16_t, 256>(p, stream);
    if (p.Dp == 128) {
        switch (dtype) {
            case 0: return launch_combine_t<float, 128>(p, stream);
            case 1: return launch_combine_t<f16_t, 128>(p, stream);
            default: return launch_combine_t<bf16_t, 128>(p, stream);
        }
    }
    switch (dtype) {
        case 0: return launch_combine_t<float, 64>(p, stream);
        case 1: return launch_combine_t<f16_t, 64>(p, stream);
        default: return launch_combine_t<bf16_t, 64>(p, stream);
    }
}

template <typename T, int D, int RMAX, int U, bool DENSE>
static hipError_t launch_decode_t(const SdpaParams& p, hipStream_t stream)
{
    constexpr int VEC = Vec16<T>::N;
    constexpr int NSTREAM = 4 * (64 / (D / VEC));
    size_t lds = (size_t)(NSTREAM * RMAX * D + NSTREAM * RMAX * 2) * sizeof(float);
    auto kern = sdpa_decode_split_kernel<T, D, RMAX, U, DENSE>;
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
    const int R = p.G * p.Sq;
    const int nchunks = (R + RMAX - 1) / RMAX;
    dim3 grid(p.num_splits, p.Hkv * nchunks, p.B);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, p);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (p.num_splits > 1) e = launch_combine_t<T, D>(p, stream);
    return e;
}

template <typename T, int D, bool DENSE>
static hipError_t launch_decode_rd(const SdpaParams& p, hipStream_t stream)
{
    const int R = p.G * p.Sq;
    if (R <= 1) return launch_decode_t<T, D, 1, 8, DENSE>(p, stream);
    if (R <= 2) return launch_decode_t<T, D, 2, 8, DENSE>(p, stream);
    if (R <= 4) return launch_decode_t<T, D, 4, 4, DENSE>(p, stream);
    return launch_decode_t<T, D, 8, 4, DENSE>(p, stream);
}

template <typename T, int D>
static hipError_t launch_decode_r(const SdpaParams& p, hipStream_t stream)
{
    return p.mask ? launch_decode_rd<T, D, true>(p, stream) : launch_decode_rd<T, D, false>(p, stream);
}

// Keys per wavefront tile for the instance launch_sdpa_decode would pick; the
// host rounds split_len to a multiple of 4 * this so splits start tile-aligned.
int decode_keys_per_tile(int dtype, int D, int R)
{
    const int vec = dtype == 0 ? 4 : 8;
    const int kpl = 64 / (D / vec);
    const int u = R <= 2 ? 8 : 4;
    return u * kpl;
}

// Host has validated: D == Dv in {64, 128}, last-dim contiguous, 16-byte aligned rows.
hipError_t launch_sdpa_decode(const SdpaParams& p, int dtype, hipStream_t stream)
{
    if (p.D == 128) {
        switch (dtype) {
            case 0: return launch_decode_r<float, 128>(p, stream);
            case 1: return launch_decode_r<f16_t, 128>(p, stream);
            default: return launch_decode_r<bf16_t, 128>(p, stream);
        }
    }
    switch (dtype) {
        case 0: return launch_decode_r<float, 64>(p, stream);
        case 1: return launch_decode_r<f16_t, 64>(p, stream);
        default: return launch_decode_r<bf16_t, 64>(p, stream);
    }
}

}  // namespace incin_rocm
