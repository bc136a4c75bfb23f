// Classifies a dense additive mask by blocks of 32 query rows x 32 keys, ahead of a matrix-core attention launch:
//   0  mixed     the block's values have to be added to the scores
//   1  zeros     every value is 0: the block needs no mask at all
//   2  hidden    every value is -inf: no key of the block is visible to any of its rows, the block is skipped
// The reference's operator knows one mask form, an additive tensor (crates/incin-backends/src/cpu/ops/shape_ops.rs:
// 1262-1266), and its callers build the causal mask as full(-inf).triu(1): with the flags, such a tensor costs about
// what the causal flag costs - blocks above the diagonal are skipped, blocks below it run the unmasked path.
// One workgroup per strip of 32 rows x 256 keys (8 blocks): a thread takes 8 consecutive keys of 4 rows - one 16-byte
// load each for 16-bit masks with unit key stride and aligned rows, element-wise loads otherwise - and the votes of a
// block meet in LDS; rows beyond Sq and keys beyond Skv do not vote.
#include "sdpa_params.h"

namespace incin_rocm {

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void mask_classify_kernel(const T* mask, int64_t m_sb, int64_t m_sh, int64_t m_si, int64_t m_sj,
                                                           int Hm, int Sq, int Skv, int nkb, uint8_t* flags, const int32_t* lims, int rows_m)
{
    __shared__ int votes[8][2];
    const int strip = blockIdx.x, rb = blockIdx.y, bh = blockIdx.z;
    if (lims != nullptr) {
        // Row limits are known (mask_row_limits_kernel ran before): the attention launches read the flags only of blocks of 128
        // or 256 rows in which some row has no limit.  If every row of the 256 around these 32 has one, nobody will ask.
        const int blk0 = (rb * 32 / 256) * 256, blk1 = min(blk0 + 256, Sq);
        const int32_t* l = lims + (int64_t)bh * rows_m;
        bool ok = true;
        for (int i = blk0 + (int)threadIdx.x; i < blk1; i += 256) ok = ok && l[rows_m > 1 ? i : 0] >= 0;
        if (__syncthreads_and(ok)) return;
    }
    const int b = bh / Hm, h = bh % Hm;
    const T* base = mask + (int64_t)b * m_sb + (int64_t)h * m_sh;
    const int c8 = threadIdx.x & 31, r0 = threadIdx.x >> 5;       // 8 keys starting at strip * 256 + c8 * 8; rows r0, r0 + 8, ..
    if (threadIdx.x < 16) votes[threadIdx.x >> 1][threadIdx.x & 1] = 0;
    __syncthreads();
    const int j0 = strip * 256 + c8 * 8;
    int not_zero = 0, not_hidden = 0;
    if (j0 < Skv) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = rb * 32 + r0 + 8 * u;
            if (i >= Sq) continue;
            const T* row = base + (int64_t)i * m_si;
            if (VEC && j0 + 7 < Skv) {
                typedef T vec8 __attribute__((ext_vector_type(8)));
                const vec8 x = *(const vec8*)(row + j0);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float f = to_f32(x[e]);
                    not_zero |= !(f == 0.0f);
                    not_hidden |= !(f == -INFINITY);
                }
            } else {
                for (int e = 0; e < 8 && j0 + e < Skv; ++e) {
                    const float f = to_f32(row[(int64_t)(j0 + e) * m_sj]);
                    not_zero |= !(f == 0.0f);
                    not_hidden |= !(f == -INFINITY);
                }
            }
        }
        if (not_zero) atomicOr(&votes[c8 >> 2][0], 1);
        if (not_hidden) atomicOr(&votes[c8 >> 2][1], 1);
    }
    __syncthreads();
    if (threadIdx.x < 8) {
        const int kb = strip * 8 + threadIdx.x;
        if (kb < nkb) flags[((int64_t)bh * gridDim.y + rb) * nkb + kb] = !votes[threadIdx.x][0] ? 1 : (!votes[threadIdx.x][1] ? 2 : 0);
    }
}

// Row limits: for every row of the mask, n if the row reads n zeros and then -inf to its end (n = Skv: all zeros, n = 0:
// all -inf), else -1.  What a causal mask, a key-padding mask and their sum look like; a kernel that knows the limit of
// every row it handles compares key numbers with it instead of reading the mask.  One wavefront per row: the first
// position that is not zero and the number of -inf values decide.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void mask_row_limits_kernel(const T* mask, int64_t m_sb, int64_t m_sh, int64_t m_si, int64_t m_sj,
                                                             int Hm, int rows_m, int Skv, int64_t n_rows, int32_t* lims)
{
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);       // (mask batch entry, mask head, row)
    if (r >= n_rows) return;
    const int i = (int)(r % rows_m);
    const int64_t bh = r / rows_m;
    const T* row = mask + (bh / Hm) * m_sb + (bh % Hm) * m_sh + (int64_t)i * m_si;
    int first = Skv, ninf = 0;
    if (VEC) {
        typedef T vec8 __attribute__((ext_vector_type(8)));
        for (int j0 = lane * 8; j0 < Skv; j0 += 512) {
            if (j0 + 7 < Skv) {
                const vec8 x = *(const vec8*)(row + j0);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float f = to_f32(x[e]);
                    if (!(f == 0.0f)) first = min(first, j0 + e);
                    ninf += f == -INFINITY;
                }
            } else {
                for (int e = 0; j0 + e < Skv; ++e) {
                    const float f = to_f32(row[j0 + e]);
                    if (!(f == 0.0f)) first = min(first, j0 + e);
                    ninf += f == -INFINITY;
                }
            }
        }
    } else {
        for (int j = lane; j < Skv; j += 64) {
            const float f = to_f32(row[(int64_t)j * m_sj]);
            if (!(f == 0.0f)) first = min(first, j);
            ninf += f == -INFINITY;
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        first = min(first, __shfl_xor(first, off, 64));
        ninf += __shfl_xor(ninf, off, 64);
    }
    if (lane == 0) lims[r] = ninf == Skv - first ? first : -1;
}

// Host has validated the extents; nbh = mask batch entries x mask heads (1 where the mask is broadcast).
hipError_t launch_mask_classify(const SdpaParams& p, int dtype, hipStream_t stream)
{
    const int nkb = (p.Skv + 31) / 32, nrb = (p.Sq + 31) / 32;
    const int Bm = p.m_sb ? p.B : 1, Hm = p.m_sh ? p.Hq : 1;
    if (nkb <= 0 || nrb <= 0) return hipSuccess;
    if (nrb > 65535 || (int64_t)Bm * Hm > 65535) return hipErrorInvalidValue;
    const dim3 grid((nkb + 7) / 8, nrb, Bm * Hm);
    uint8_t* flags = (uint8_t*)p.mask_flags;
    const int esz = dtype == 0 ? 4 : 2;
    // 8 consecutive elements in one vector load: unit key stride, every row start a multiple of the vector
    const bool vec = p.m_sj == 1 && ((uintptr_t)p.mask % (8 * esz)) == 0 && p.m_sb % 8 == 0 && p.m_sh % 8 == 0 && p.m_si % 8 == 0;
    const int rows_m = p.m_si ? p.Sq : 1;
    if (p.mask_lims) {       // the limits first: the flags of blocks whose rows all have one are not needed
        const int64_t n_rows = (int64_t)Bm * Hm * rows_m;
        const dim3 lgrid((unsigned)((n_rows + 3) / 4));
#define LIMITS(T, V) hipLaunchKernelGGL((mask_row_limits_kernel<T, V>), lgrid, dim3(256), 0, stream, (const T*)p.mask, p.m_sb, p.m_sh, p.m_si, p.m_sj, Hm, rows_m, p.Skv, n_rows, (int32_t*)p.mask_lims)
        switch (dtype) {
            case 0: if (vec) LIMITS(float, true); else LIMITS(float, false); break;
            case 1: if (vec) LIMITS(f16_t, true); else LIMITS(f16_t, false); break;
            default: if (vec) LIMITS(bf16_t, true); else LIMITS(bf16_t, false); break;
        }
#undef LIMITS
    }
#define CLASSIFY(T, V) hipLaunchKernelGGL((mask_classify_kernel<T, V>), grid, dim3(256), 0, stream, (const T*)p.mask, p.m_sb, p.m_sh, p.m_si, p.m_sj, Hm, p.Sq, p.Skv, nkb, flags, p.mask_lims, rows_m)
    switch (dtype) {
        case 0: if (vec) CLASSIFY(float, true); else CLASSIFY(float, false); break;
        case 1: if (vec) CLASSIFY(f16_t, true); else CLASSIFY(f16_t, false); break;
        default: if (vec) CLASSIFY(bf16_t, true); else CLASSIFY(bf16_t, false); break;
    }
#undef CLASSIFY
    return hipGetLastError();
}

// The row limits of a mask given by itself: shape [A0, A1, rows, Skv] with element strides (0 where an axis is repeated),
// one int per (a0, a1, row) in that order.  Behind incin_rocm_mask_row_limits.
hipError_t launch_mask_row_limits(const void* mask, int dtype, const int64_t shape[4], const int64_t strides[4], int32_t* lims, hipStream_t stream)
{
    const int64_t n_rows = shape[0] * shape[1] * shape[2];
    if (n_rows <= 0) return hipSuccess;
    if ((n_rows + 3) / 4 > 0x7fffffffLL) return hipErrorInvalidValue;
    const dim3 grid((unsigned)((n_rows + 3) / 4));
    const int esz = dtype == 0 ? 4 : 2;
    const bool vec = strides[3] == 1 && ((uintptr_t)mask % (8 * esz)) == 0 && strides[0] % 8 == 0 && strides[1] % 8 == 0 && strides[2] % 8 == 0;
#define LIMITS(T, V) hipLaunchKernelGGL((mask_row_limits_kernel<T, V>), grid, dim3(256), 0, stream, (const T*)mask, strides[0], strides[1], strides[2], strides[3], (int)shape[1], (int)shape[2], (int)shape[3], n_rows, lims)
    switch (dtype) {
        case 0: if (vec) LIMITS(float, true); else LIMITS(float, false); break;
        case 1: if (vec) LIMITS(f16_t, true); else LIMITS(f16_t, false); break;
        default: if (vec) LIMITS(bf16_t, true); else LIMITS(bf16_t, false); break;
    }
#undef LIMITS
    return hipGetLastError();
}

}  // namespace incin_rocm
