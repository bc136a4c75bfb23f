// Generic attention backward: fp32 FMA arithmetic, any of f32/f16/bf16 storage, D and Dv up to DMAX, dense additive
// mask + causal + per-batch key lengths.  The kernel every backward request can fall back on (the reference's own
// dtype, f32, comes through here); the MFMA kernels of sdpa_bwd_mfma.hip cover f16/bf16 at D = 128.
//
// The gradients are those of the reference's taped composition (crates/incin-backends/src/cpu/ops/shape_ops.rs:1245-1269
// walked by cpu/tape.rs:149-176; matmul rule cpu/ops/matmul.rs:264-281, log-softmax chain cpu/ops/elementwise.rs:1062-1077):
//
//   x_ij = s q_i.k_j + mask_ij     P_ij = exp(x_ij - L_i)     dP_ij = dO_i . V_j     D_i = dO_i . O_i
//   dS_ij = P_ij (dP_ij - D_i)     dV_j = sum_i P_ij dO_i     dK_j = s sum_i dS_ij Q_i     dQ_i = s sum_j dS_ij K_j
//
// with L_i the forward's row normaliser.  Three kernels, no atomics:
//   bwd_generic_delta_kernel   D_i into the workspace
//   bwd_generic_dq_kernel      a workgroup (16 x 16 threads) owns 32 query rows and walks the keys 32 at a time
//   bwd_generic_dkv_kernel     a workgroup owns 32 keys and walks the query rows of the group's heads 32 at a time
// Tiles live in LDS as f32 with one float of row padding.  In a 32 x 32 tile of S / dP, thread (ty, tx) owns rows
// 2*ty, 2*ty + 1 and columns tx, tx + 16; of an accumulator tile the same rows and columns tx + 16*c.
// A query row without a visible key (L_i = -inf; NaN in the forward) contributes nothing and gets a zero dQ.
#include "sdpa_bwd.h"

namespace incin_rocm {

constexpr int GB = 32;      // rows and columns of a score tile

template <typename T>
__global__ __launch_bounds__(256) void bwd_generic_delta_kernel(SdpaBwdParams p)
{
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);     // (b * Hq + hq) * Sq + i
    const int64_t rows = (int64_t)p.f.B * p.f.Hq * p.f.Sq;
    if (row >= rows) return;
    const int i = (int)(row % p.f.Sq);
    const int64_t bh = row / p.f.Sq;
    const int hq = (int)(bh % p.f.Hq), b = (int)(bh / p.f.Hq);
    const T* o = (const T*)p.f.o + b * p.f.o_sb + hq * p.f.o_sh + (int64_t)i * p.f.o_ss;
    const T* g = (const T*)p.d_o + b * p.do_sb + hq * p.do_sh + (int64_t)i * p.do_ss;
    float acc = 0.0f;
    for (int d = lane; d < p.f.Dv; d += 64) acc = fmaf(to_f32(o[d]), to_f32(g[d]), acc);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane == 0) p.neg_delta[row] = p.f.lse[row] == -INFINITY ? 0.0f : -acc;
}

// rows [r0, r0 + 32) of a [rows, n] tensor (row stride `stride` elements) into dst[32][pitch] as f32, zeros past the end
template <typename T>
__device__ __forceinline__ void load_tile(float* dst, int pitch, const T* base, int64_t stride, int r0, int rows, int n, int tid)
{
    for (int idx = tid; idx < GB * n; idx += 256) {
        const int r = idx / n, d = idx - r * n;
        const int row = r0 + r;
        dst[r * pitch + d] = row < rows ? to_f32(base[(int64_t)row * stride + d]) : 0.0f;
    }
}

// P and dS of one (query i, key j) pair from the raw products s = q_i.k_j and dp = dO_i.v_j
struct Pair { float p, ds; };
template <typename T>
__device__ __forceinline__ Pair pair_of(const SdpaParams& f, int rows_b, const T* mp, int i, int j, int kv_len, int coff, float s, float dp, float L, float negD)
{
    Pair r = {0.0f, 0.0f};
    if (i >= rows_b || j >= kv_len || (f.causal && j > i + coff) || L == -INFINITY) return r;
    float x = s * f.scale;
    if (mp) x += to_f32(mp[(int64_t)i * f.m_si + (int64_t)j * f.m_sj]);
    if (x == -INFINITY) return r;         // hidden by the dense mask
    r.p = expf(x - L);
    r.ds = r.p * (dp + negD);
    return r;
}

template <typename T, int DMAX>
__global__ __launch_bounds__(256) void bwd_generic_dq_kernel(SdpaBwdParams bp)
{
    constexpr int DP = DMAX + 1, NC = DMAX / 16;
    const SdpaParams& p = bp.f;
    extern __shared__ float smem[];
    float* Qs = smem;                    // [32][DP]
    float* Gs = Qs + GB * DP;            // dO
    float* Ks = Gs + GB * DP;
    float* Vs = Ks + GB * DP;
    float* Ss = Vs + GB * DP;            // dS, [32][33]

    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int q0 = blockIdx.x * GB, hq = blockIdx.y, b = blockIdx.z;
    const int hkv = hq / p.G;
    const int D = p.D, Dv = p.Dv, Sq = p.Sq, Skv = p.Skv;
    const T* qp = (const T*)p.q + (int64_t)b * p.q_sb + (int64_t)hq * p.q_sh;
    const T* kp = (const T*)p.k + (int64_t)b * p.k_sb + (int64_t)hkv * p.k_sh;
    const T* vp = (const T*)p.v + (int64_t)b * p.v_sb + (int64_t)hkv * p.v_sh;
    const T* gp = (const T*)bp.d_o + (int64_t)b * bp.do_sb + (int64_t)hq * bp.do_sh;
    T* dqp = (T*)bp.d_q + (int64_t)b * bp.dq_sb + (int64_t)hq * bp.dq_sh;
    const T* mp = p.mask ? (const T*)p.mask + (int64_t)b * p.m_sb + (int64_t)hq * p.m_sh : nullptr;

    // query rows at and beyond rows_b are padding (q_lens): they arrive as zeros, weigh nothing and get a zero dQ
    const int rows_b = p.q_lens ? clampi(p.q_lens[b], 0, Sq) : Sq;
    load_tile(Qs, DP, qp, p.q_ss, q0, rows_b, D, tid);
    load_tile(Gs, DP, gp, bp.do_ss, q0, rows_b, Dv, tid);

    int kv_len = Skv;
    if (p.kv_lens) kv_len = clampi(p.kv_lens[b], 0, Skv);
    const int coff = Skv - Sq;
    int j_end = kv_len;
    if (p.causal) j_end = clampi(min(q0 + GB - 1, Sq - 1) + coff + 1, 0, kv_len);
    if (q0 >= rows_b) j_end = 0;

    float L[2], negD[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const int i = min(q0 + 2 * ty + r, Sq - 1);
        const int64_t stat = ((int64_t)b * p.Hq + hq) * Sq + i;
        L[r] = p.lse[stat];
        negD[r] = bp.neg_delta[stat];
    }
    float acc[2][NC];
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int c = 0; c < NC; ++c) acc[r][c] = 0.0f;

    for (int j0 = 0; j0 < j_end; j0 += GB) {
        __syncthreads();                         // the previous tile is consumed (and Q, dO are stored)
        load_tile(Ks, DP, kp, p.k_ss, j0, Skv, D, tid);
        load_tile(Vs, DP, vp, p.v_ss, j0, Skv, Dv, tid);
        __syncthreads();
        float s[2][2] = {{0.0f, 0.0f}, {0.0f, 0.0f}}, dp[2][2] = {{0.0f, 0.0f}, {0.0f, 0.0f}};
        for (int d = 0; d < D; ++d) {
            const float q0v = Qs[(2 * ty) * DP + d], q1v = Qs[(2 * ty + 1) * DP + d];
            const float k0v = Ks[tx * DP + d], k1v = Ks[(tx + 16) * DP + d];
            s[0][0] = fmaf(q0v, k0v, s[0][0]); s[0][1] = fmaf(q0v, k1v, s[0][1]);
            s[1][0] = fmaf(q1v, k0v, s[1][0]); s[1][1] = fmaf(q1v, k1v, s[1][1]);
        }
        for (int d = 0; d < Dv; ++d) {
            const float g0v = Gs[(2 * ty) * DP + d], g1v = Gs[(2 * ty + 1) * DP + d];
            const float v0v = Vs[tx * DP + d], v1v = Vs[(tx + 16) * DP + d];
            dp[0][0] = fmaf(g0v, v0v, dp[0][0]); dp[0][1] = fmaf(g0v, v1v, dp[0][1]);
            dp[1][0] = fmaf(g1v, v0v, dp[1][0]); dp[1][1] = fmaf(g1v, v1v, dp[1][1]);
        }
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int c = 0; c < 2; ++c)
                Ss[(2 * ty + r) * (GB + 1) + tx + 16 * c] =
                    pair_of(p, rows_b, mp, q0 + 2 * ty + r, j0 + tx + 16 * c, kv_len, coff, s[r][c], dp[r][c], L[r], negD[r]).ds;
        __syncthreads();
        for (int jj = 0; jj < GB; ++jj) {
            const float d0 = Ss[(2 * ty) * (GB + 1) + jj], d1 = Ss[(2 * ty + 1) * (GB + 1) + jj];
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const float kv = Ks[jj * DP + tx + 16 * c];      // (columns past D hold what the previous user left: not stored below)
                acc[0][c] = fmaf(d0, kv, acc[0][c]);
                acc[1][c] = fmaf(d1, kv, acc[1][c]);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const int i = q0 + 2 * ty + r;
        if (i >= Sq) continue;
#pragma unroll
        for (int c = 0; c < NC; ++c)
            if (tx + 16 * c < D) dqp[(int64_t)i * bp.dq_ss + tx + 16 * c] = from_f32<T>(i < rows_b ? acc[r][c] * p.scale : 0.0f);
    }
}

template <typename T, int DMAX>
__global__ __launch_bounds__(256) void bwd_generic_dkv_kernel(SdpaBwdParams bp)
{
    constexpr int DP = DMAX + 1, NC = DMAX / 16;
    const SdpaParams& p = bp.f;
    extern __shared__ float smem[];
    float* Ks = smem;                    // [32][DP]
    float* Vs = Ks + GB * DP;
    float* Qs = Vs + GB * DP;
    float* Gs = Qs + GB * DP;            // dO
    float* Ps = Gs + GB * DP;            // P^T, [key][query], [32][33]
    float* Ss = Ps + GB * (GB + 1);      // dS^T
    float* Ls = Ss + GB * (GB + 1);      // L_i of the tile's rows, then -D_i
    float* Ds = Ls + GB;

    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int j0 = blockIdx.x * GB, hkv = blockIdx.y, b = blockIdx.z;
    const int D = p.D, Dv = p.Dv, Sq = p.Sq, Skv = p.Skv;
    const T* kp = (const T*)p.k + (int64_t)b * p.k_sb + (int64_t)hkv * p.k_sh;
    const T* vp = (const T*)p.v + (int64_t)b * p.v_sb + (int64_t)hkv * p.v_sh;
    T* dkp = (T*)bp.d_k + (int64_t)b * bp.dk_sb + (int64_t)hkv * bp.dk_sh;
    T* dvp = (T*)bp.d_v + (int64_t)b * bp.dv_sb + (int64_t)hkv * bp.dv_sh;

    load_tile(Ks, DP, kp, p.k_ss, j0, Skv, D, tid);
    load_tile(Vs, DP, vp, p.v_ss, j0, Skv, Dv, tid);

    int kv_len = Skv;
    if (p.kv_lens) kv_len = clampi(p.kv_lens[b], 0, Skv);
    const int coff = Skv - Sq;
    // first query row that sees a key of this block (causal: i >= j - coff)
    const int i_begin = p.causal ? clampi(j0 - coff, 0, Sq) / GB * GB : 0;
    const int rows_b = p.q_lens ? clampi(p.q_lens[b], 0, Sq) : Sq;      // query rows at and beyond are padding (q_lens)
    const int i_end = j0 < kv_len ? rows_b : 0;

    float dk[2][NC], dv[2][NC];
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int c = 0; c < NC; ++c) { dk[r][c] = 0.0f; dv[r][c] = 0.0f; }

    for (int gq = 0; gq < p.G; ++gq) {
        const int hq = hkv * p.G + gq;
        const T* qp = (const T*)p.q + (int64_t)b * p.q_sb + (int64_t)hq * p.q_sh;
        const T* gp = (const T*)bp.d_o + (int64_t)b * bp.do_sb + (int64_t)hq * bp.do_sh;
        const T* mp = p.mask ? (const T*)p.mask + (int64_t)b * p.m_sb + (int64_t)hq * p.m_sh : nullptr;
        const int64_t stat0 = ((int64_t)b * p.Hq + hq) * Sq;
        for (int i0 = i_begin; i0 < i_end; i0 += GB) {
            __syncthreads();                     // the previous tile is consumed (and K, V are stored)
            load_tile(Qs, DP, qp, p.q_ss, i0, rows_b, D, tid);
            load_tile(Gs, DP, gp, bp.do_ss, i0, rows_b, Dv, tid);
            if (tid < GB) {
                const int i = min(i0 + tid, Sq - 1);
                Ls[tid] = p.lse[stat0 + i];
                Ds[tid] = bp.neg_delta[stat0 + i];
            }
            __syncthreads();
            // thread (ty, tx): keys 2*ty, 2*ty + 1 and queries tx, tx + 16
            float s[2][2] = {{0.0f, 0.0f}, {0.0f, 0.0f}}, dp[2][2] = {{0.0f, 0.0f}, {0.0f, 0.0f}};
            for (int d = 0; d < D; ++d) {
                const float k0v = Ks[(2 * ty) * DP + d], k1v = Ks[(2 * ty + 1) * DP + d];
                const float q0v = Qs[tx * DP + d], q1v = Qs[(tx + 16) * DP + d];
                s[0][0] = fmaf(k0v, q0v, s[0][0]); s[0][1] = fmaf(k0v, q1v, s[0][1]);
                s[1][0] = fmaf(k1v, q0v, s[1][0]); s[1][1] = fmaf(k1v, q1v, s[1][1]);
            }
            for (int d = 0; d < Dv; ++d) {
                const float v0v = Vs[(2 * ty) * DP + d], v1v = Vs[(2 * ty + 1) * DP + d];
                const float g0v = Gs[tx * DP + d], g1v = Gs[(tx + 16) * DP + d];
                dp[0][0] = fmaf(v0v, g0v, dp[0][0]); dp[0][1] = fmaf(v0v, g1v, dp[0][1]);
                dp[1][0] = fmaf(v1v, g0v, dp[1][0]); dp[1][1] = fmaf(v1v, g1v, dp[1][1]);
            }
#pragma unroll
            for (int r = 0; r < 2; ++r)
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    const int ii = tx + 16 * c;
                    const Pair pr = pair_of(p, rows_b, mp, i0 + ii, j0 + 2 * ty + r, kv_len, coff, s[r][c], dp[r][c], Ls[ii], Ds[ii]);
                    Ps[(2 * ty + r) * (GB + 1) + ii] = pr.p;
                    Ss[(2 * ty + r) * (GB + 1) + ii] = pr.ds;
                }
            __syncthreads();
            for (int ii = 0; ii < GB; ++ii) {
                const float p0 = Ps[(2 * ty) * (GB + 1) + ii], p1 = Ps[(2 * ty + 1) * (GB + 1) + ii];
                const float s0 = Ss[(2 * ty) * (GB + 1) + ii], s1 = Ss[(2 * ty + 1) * (GB + 1) + ii];
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    const float gv = Gs[ii * DP + tx + 16 * c], qv = Qs[ii * DP + tx + 16 * c];
                    dv[0][c] = fmaf(p0, gv, dv[0][c]); dv[1][c] = fmaf(p1, gv, dv[1][c]);
                    dk[0][c] = fmaf(s0, qv, dk[0][c]); dk[1][c] = fmaf(s1, qv, dk[1][c]);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const int j = j0 + 2 * ty + r;
        if (j >= Skv) continue;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int col = tx + 16 * c;
            if (col < D) dkp[(int64_t)j * bp.dk_ss + col] = from_f32<T>(dk[r][c] * p.scale);
            if (col < Dv) dvp[(int64_t)j * bp.dv_ss + col] = from_f32<T>(dv[r][c]);
        }
    }
}

template <typename T, int DMAX>
static hipError_t launch_bwd_generic_t(const SdpaBwdParams& bp, hipStream_t stream)
{
    const SdpaParams& p = bp.f;
    const int64_t rows = (int64_t)p.B * p.Hq * p.Sq;
    const size_t tile = (size_t)GB * (DMAX + 1) * sizeof(float), sq = (size_t)GB * (GB + 1) * sizeof(float);
    if (rows > 0) {
        hipLaunchKernelGGL((bwd_generic_delta_kernel<T>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, bp);
        const size_t lds = 4 * tile + sq;
        auto kern = bwd_generic_dq_kernel<T, DMAX>;
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3((p.Sq + GB - 1) / GB, p.Hq, p.B), dim3(256), lds, stream, bp);
    }
    if ((int64_t)p.B * p.Hkv * p.Skv > 0) {
        const size_t lds = 4 * tile + 2 * sq + 2 * GB * sizeof(float);
        auto kern = bwd_generic_dkv_kernel<T, DMAX>;
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3((p.Skv + GB - 1) / GB, p.Hkv, p.B), dim3(256), lds, stream, bp);
    }
    return hipGetLastError();
}

template <typename T>
static hipError_t launch_bwd_generic_d(const SdpaBwdParams& bp, hipStream_t stream)
{
    const int dm = bp.f.D > bp.f.Dv ? bp.f.D : bp.f.Dv;
    if (dm <= 64) return launch_bwd_generic_t<T, 64>(bp, stream);
    if (dm <= 128) return launch_bwd_generic_t<T, 128>(bp, stream);
    return launch_bwd_generic_t<T, 256>(bp, stream);
}

// dtype: 0 f32, 1 f16, 2 bf16.  Host has validated max(D, Dv) <= 256, unit last-axis strides, lse and the workspace present.
hipError_t launch_sdpa_bwd_generic(const SdpaBwdParams& bp, int dtype, hipStream_t stream)
{
    switch (dtype) {
        case 0: return launch_bwd_generic_d<float>(bp, stream);
        case 1: return launch_bwd_generic_d<f16_t>(bp, stream);
        default: return launch_bwd_generic_d<bf16_t>(bp, stream);
    }
}

}  // namespace incin_rocm
