// Classifies a dense additive mask by blocks of 32 query rows x 32 keys, ahead of a matrix-core attention launch:
//   0  mixed     the block's values have to be added to the scores
//   1  zeros     every value is 0: the block needs no mask at all
//   2  hidden    every value is -inf: no key of the block is visible to any of its rows, the block is skipped
// The reference's operator knows one mask form, an additive tensor (crates/incin-backends/src/cpu/ops/shape_ops.rs:
// 1262-1266), and its callers build the causal mask as full(-inf).triu(1): with the flags, such a tensor costs about
// what the causal flag costs - blocks above the diagonal are skipped, blocks below it run the unmasked path.
// One workgroup per block: 1024 elements, 4 per thread; rows beyond Sq and keys beyond Skv do not vote.
#include "sdpa_params.h"

namespace incin_rocm {

template <typename T>
__global__ __launch_bounds__(256) void mask_classify_kernel(const T* mask, int64_t m_sb, int64_t m_sh, int64_t m_si, int64_t m_sj,
                                                           int Hm, int Sq, int Skv, uint8_t* flags)
{
    const int kb = blockIdx.x, rb = blockIdx.y, bh = blockIdx.z;
    const int b = bh / Hm, h = bh % Hm;
    const T* base = mask + (int64_t)b * m_sb + (int64_t)h * m_sh;
    const int c = threadIdx.x & 31, r0 = threadIdx.x >> 5;
    const int j = kb * 32 + c;
    int not_zero = 0, not_hidden = 0;
    if (j < Skv) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = rb * 32 + r0 + 8 * u;
            if (i < Sq) {
                const float x = to_f32(base[(int64_t)i * m_si + (int64_t)j * m_sj]);
                not_zero |= !(x == 0.0f);
                not_hidden |= !(x == -INFINITY);
            }
        }
    }
    not_zero = __syncthreads_or(not_zero);
    not_hidden = __syncthreads_or(not_hidden);
    if (threadIdx.x == 0)
        flags[((int64_t)bh * gridDim.y + rb) * gridDim.x + kb] = !not_zero ? 1 : (!not_hidden ? 2 : 0);
}

// Host has validated the extents; nbh = mask batch entries x mask heads (1 where the mask is broadcast).
hipError_t launch_mask_classify(const SdpaParams& p, int dtype, hipStream_t stream)
{
    const int nkb = (p.Skv + 31) / 32, nrb = (p.Sq + 31) / 32;
    const int Bm = p.m_sb ? p.B : 1, Hm = p.m_sh ? p.Hq : 1;
    if (nkb <= 0 || nrb <= 0) return hipSuccess;
    if (nrb > 65535 || (int64_t)Bm * Hm > 65535) return hipErrorInvalidValue;
    const dim3 grid(nkb, nrb, Bm * Hm);
    uint8_t* flags = (uint8_t*)p.mask_flags;
    switch (dtype) {
        case 0: hipLaunchKernelGGL(mask_classify_kernel<float>, grid, dim3(256), 0, stream, (const float*)p.mask, p.m_sb, p.m_sh, p.m_si, p.m_sj, Hm, p.Sq, p.Skv, flags); break;
        case 1: hipLaunchKernelGGL(mask_classify_kernel<f16_t>, grid, dim3(256), 0, stream, (const f16_t*)p.mask, p.m_sb, p.m_sh, p.m_si, p.m_sj, Hm, p.Sq, p.Skv, flags); break;
        default: hipLaunchKernelGGL(mask_classify_kernel<bf16_t>, grid, dim3(256), 0, stream, (const bf16_t*)p.mask, p.m_sb, p.m_sh, p.m_si, p.m_sj, Hm, p.Sq, p.Skv, flags); break;
    }
    return hipGetLastError();
}

}  // namespace incin_rocm
