// Device-to-device copy as a plain kernel: 16 bytes per lane per iteration,
// grid-stride.  Backs incin_rocm_memcpy_d2d for 16-byte aligned buffers; being
// an ordinary dispatch of known size it is also what hardware byte counters
// are calibrated against.
#include <hip/hip_runtime.h>
#include <stdint.h>

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
