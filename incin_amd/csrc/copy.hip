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
