// Device-to-device copy as a plain kernel: 16 bytes per lane per iteration,
// grid-stride.  Backs incin_rocm_memcpy_d2d for 16-byte aligned buffers; being
// an ordinary dispatch of known size it is also what hardware byte counters
// are calibrated against.
#include "copy.h"

namespace incin_rocm {

typedef unsigned int uint4v __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void copy16_kernel(const uint4v* __restrict__ src, uint4v* __restrict__ dst, size_t n16)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

hipError_t launch_copy16(void* dst, const void* src, size_t bytes, hipStream_t stream)
{
    const size_t n16 = bytes / 16;
    if (n16 == 0) return hipSuccess;
    size_t blocks = (n16 + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    hipLaunchKernelGGL(copy16_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint4v*)src, (uint4v*)dst, n16);
    return hipGetLastError();
}

}  // namespace incin_rocm

// ---- strided view -> contiguous buffer ----------------------------------------------------------------------------
// What the reference's CpuStorage::contiguous does element by element on the host
// (crates/incin-backends/src/cpu/storage.rs:407-440): the logical (row-major) contents of a view with arbitrary
// element strides, written densely.  A workgroup moves one 32 x 32 tile of the last two axes through LDS: it reads
// along whichever of the two axes has the smaller source stride and writes along the last axis, so both sides touch
// memory in runs (a transposed view is the case that matters: the operator's K arrives as transpose([.., D, S])).
namespace incin_rocm {

template <typename E>
__global__ __launch_bounds__(256) void copy_strided_kernel(StridedCopyParams p)
{
    __shared__ E tile[32][33];
    const int64_t R = p.shape[6], C = p.shape[7];
    const int64_t sr = p.stride[6], sc = p.stride[7];
    const int64_t tiles_c = (C + 31) / 32;
    const int64_t r0 = (int64_t)(blockIdx.x / tiles_c) * 32, c0 = (int64_t)(blockIdx.x % tiles_c) * 32;
    // the outer index of this workgroup -> source offset of its [R, C] slice
    int64_t o = (int64_t)blockIdx.y + (int64_t)blockIdx.z * 65535, src_off = 0;
    if (o >= p.outer) return;
    const int64_t dst_off = o * R * C;
#pragma unroll
    for (int a = 5; a >= 0; --a) {
        const int64_t n = p.shape[a];
        src_off += (o % n) * p.stride[a];
        o /= n;
    }
    const E* src = (const E*)p.src + src_off;
    E* dst = (E*)p.dst + dst_off;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const bool along_rows = (sr < 0 ? -sr : sr) < (sc < 0 ? -sc : sc);      // the source runs along the row axis
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int a = ty + 8 * i;
        const int64_t r = along_rows ? r0 + tx : r0 + a, c = along_rows ? c0 + a : c0 + tx;
        if (r < R && c < C) tile[r - r0][c - c0] = src[r * sr + c * sc];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t r = r0 + ty + 8 * i, c = c0 + tx;
        if (r < R && c < C) dst[r * C + c] = tile[r - r0][c - c0];
    }
}

hipError_t launch_copy_strided(const StridedCopyParams& p, hipStream_t stream)
{
    const int64_t R = p.shape[6], C = p.shape[7];
    if (p.outer <= 0 || R <= 0 || C <= 0) return hipSuccess;
    const int64_t tiles = ((R + 31) / 32) * ((C + 31) / 32);
    if (tiles > 0x7fffffffLL || p.outer > 65535LL * 65535LL) return hipErrorInvalidValue;
    const dim3 grid((unsigned)tiles, (unsigned)(p.outer < 65535 ? p.outer : 65535), (unsigned)((p.outer + 65534) / 65535));
    if (p.elem == 2) hipLaunchKernelGGL(copy_strided_kernel<uint16_t>, grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(copy_strided_kernel<uint32_t>, grid, dim3(256), 0, stream, p);
    return hipGetLastError();
}

// Zero-fills rows [B, H, S, row_elems] addressed by element strides (a kernel rather than a memset: it may be recorded
// into a launch graph).
template <typename E>
__global__ __launch_bounds__(256) void zero_rows_kernel(E* base, int64_t sb, int64_t sh, int64_t ss, int S, int row_elems)
{
    const int64_t rows = (int64_t)S * gridDim.y * gridDim.z;
    (void)rows;
    E* bh = base + (int64_t)blockIdx.z * sb + (int64_t)blockIdx.y * sh;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < (int64_t)S * row_elems; i += (int64_t)gridDim.x * blockDim.x)
        bh[(i / row_elems) * ss + (i % row_elems)] = (E)0;
}

hipError_t launch_zero_rows(void* base, int elem, int B, int H, int S, int row_elems, int64_t sb, int64_t sh, int64_t ss, hipStream_t stream)
{
    if (B <= 0 || H <= 0 || S <= 0 || row_elems <= 0) return hipSuccess;
    int64_t blocks = ((int64_t)S * row_elems + 255) / 256;
    if (blocks > 1024) blocks = 1024;
    const dim3 grid((unsigned)blocks, (unsigned)H, (unsigned)B);
    if (elem == 2) hipLaunchKernelGGL(zero_rows_kernel<uint16_t>, grid, dim3(256), 0, stream, (uint16_t*)base, sb, sh, ss, S, row_elems);
    else hipLaunchKernelGGL(zero_rows_kernel<uint32_t>, grid, dim3(256), 0, stream, (uint32_t*)base, sb, sh, ss, S, row_elems);
    return hipGetLastError();
}

}  // namespace incin_rocm

// ---- gradient of a broadcast: sums over the axes an operand was repeated along -------------------------------------
// What the reference's tape does with the gradient of a broadcast operand (crates/incin-backends/src/cpu/tape.rs:
// 243-265, `unbroadcast`, through `sum_dim_keepdim`, :283-317): the axes along which the operand had extent 1 are summed
// away, one axis after the other from the left, each sum running over the axis in ascending order from 0.  One thread
// per destination element keeps that order (a partial sum per reduced axis, folded into the next axis's when the axis
// wraps), so the f32 result has the reference's rounding sequence; 16-bit storage is summed in f32 and rounded once
// (the reference rounds after every addition).
namespace incin_rocm {

template <int DT> struct SumElem;
template <> struct SumElem<0> { typedef float T; static __device__ float load(const T* p) { return *p; } static __device__ void store(T* p, float v) { *p = v; } };
template <> struct SumElem<1> { typedef _Float16 T; static __device__ float load(const T* p) { return (float)*p; } static __device__ void store(T* p, float v) { *p = (T)v; } };
template <> struct SumElem<2> { typedef __bf16 T; static __device__ float load(const T* p) { return (float)*p; } static __device__ void store(T* p, float v) { *p = (T)v; } };

template <int DT>
__global__ __launch_bounds__(256) void sum_to_shape_kernel(SumToShapeParams p, int64_t n_dst)
{
    typedef typename SumElem<DT>::T T;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_dst) return;
    // destination index -> source offset of its first term; the reduced axes, leftmost first
    int64_t sstride[8], acc_s = 1;
#pragma unroll
    for (int a = 7; a >= 0; --a) { sstride[a] = acc_s; acc_s *= p.src_shape[a]; }
    int64_t off = 0, rem = i;
#pragma unroll
    for (int a = 7; a >= 0; --a) {
        const int64_t n = p.dst_shape[a];
        off += (rem % n) * sstride[a];
        rem /= n;
    }
    int64_t rext[8], rstr[8];
    int nred = 0;
#pragma unroll
    for (int a = 0; a < 8; ++a)
        if (p.dst_shape[a] != p.src_shape[a]) { rext[nred] = p.src_shape[a]; rstr[nred] = sstride[a]; ++nred; }
    const T* src = (const T*)p.src;
    if (nred == 0) { SumElem<DT>::store((T*)p.dst + i, SumElem<DT>::load(src + off)); return; }
    float acc[8];
    int64_t idx[8];
    for (int l = 0; l < 8; ++l) { acc[l] = 0.0f; idx[l] = 0; }
    for (;;) {
        acc[0] += SumElem<DT>::load(src + off);
        int l = 0;
        bool done = false;
        for (;;) {
            off += rstr[l];
            if (++idx[l] < rext[l]) break;
            off -= rstr[l] * rext[l];
            idx[l] = 0;
            if (l + 1 == nred) { done = true; break; }
            acc[l + 1] += acc[l];
            acc[l] = 0.0f;
            ++l;
        }
        if (done) break;
    }
    SumElem<DT>::store((T*)p.dst + i, acc[nred - 1]);
}

hipError_t launch_sum_to_shape(const SumToShapeParams& p, hipStream_t stream)
{
    int64_t n_dst = 1;
    for (int a = 0; a < 8; ++a) n_dst *= p.dst_shape[a];
    if (n_dst <= 0) return hipSuccess;
    const int64_t blocks = (n_dst + 255) / 256;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    switch (p.dtype) {
        case 0: hipLaunchKernelGGL(sum_to_shape_kernel<0>, dim3((unsigned)blocks), dim3(256), 0, stream, p, n_dst); break;
        case 1: hipLaunchKernelGGL(sum_to_shape_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, stream, p, n_dst); break;
        default: hipLaunchKernelGGL(sum_to_shape_kernel<2>, dim3((unsigned)blocks), dim3(256), 0, stream, p, n_dst); break;
    }
    return hipGetLastError();
}

}  // namespace incin_rocm
