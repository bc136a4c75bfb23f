// Diagnostic kernel behind incin_rocm_matrix_rate: what rate of bf16 matrix instructions this device sustains, as a function of
// the DATA the instructions work on.  No counterpart in the reference; it exists because the bound of the 16-bit attention
// kernels on this hardware is not a pipe but the power the chip may draw: a loop of nothing but v_mfma_f32_32x32x16_bf16 runs
// near the nominal peak on zeros and about a third slower on random values, and the attention kernels sit under the second
// figure.  bench.py reports both beside the roofline of the prefill kernel.
#include <hip/hip_runtime.h>

#include "sdpa_mfma_common.h"

namespace incin_rocm {

// MIX 0: matrix instructions only.  MIX 1: per matrix instruction two v_exp_f32, three other vector instructions and one
// 16-byte LDS read - the instruction mix of the prefill kernel's pipelined loop - all independent of the products.
// 512 threads: two wavefronts per SIMD.  Operands: 16 bytes per lane and operand from `src` (64 Ki dwords, whatever they hold).
template <int MIX>
__global__ __launch_bounds__(512) void matrix_rate_kernel(const unsigned* __restrict__ src, float* __restrict__ sink, int iterations)
{
    __shared__ unsigned lds[16 * 1024];
    union { bf16x8 v; unsigned u[4]; } a[4], b[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            a[j].u[e] = src[(threadIdx.x * 16 + j * 4 + e) & 65535];
            b[j].u[e] = src[(threadIdx.x * 16 + 7 + j * 4 + e + 32768) & 65535];
        }
    for (int i = threadIdx.x; i < 16 * 1024; i += blockDim.x) lds[i] = src[i];
    __syncthreads();
    floatx16 c[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) c[j][r] = 0.0f;
    float v[12], t[8];
#pragma unroll
    for (int i = 0; i < 12; ++i) v[i] = threadIdx.x * 0.001f + i;
#pragma unroll
    for (int i = 0; i < 8; ++i) t[i] = -(threadIdx.x * 0.01f) - i;
    const unsigned laddr = lds_address(lds) + (threadIdx.x & 63) * 16;
    float4 ld[4] = {};
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            c[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j].v, b[j].v, c[j], 0, 0, 0);
            if (MIX == 1) {
                t[2 * j] = __builtin_amdgcn_exp2f(t[2 * j]);
                v[3 * j] = __builtin_fmaf(v[3 * j], 1.0001f, 0.5f);
                t[2 * j + 1] = __builtin_amdgcn_exp2f(t[2 * j + 1]);
                v[3 * j + 1] = __builtin_fmaf(v[3 * j + 1], 1.0001f, 0.5f);
                v[3 * j + 2] = __builtin_fmaf(v[3 * j + 2], 1.0001f, 0.5f);
                asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(ld[j]) : "v"(laddr), "n"(j * 1024));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (MIX == 1) asm volatile("s_waitcnt lgkmcnt(0)");
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 12; ++i) s += v[i];
#pragma unroll
    for (int i = 0; i < 8; ++i) s += t[i];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        s += ld[j].x + ld[j].w;
#pragma unroll
        for (int r = 0; r < 16; ++r) s += c[j][r];
    }
    sink[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// One workgroup per compute unit; `src` holds 256 KiB, `sink` takes 4 bytes per thread (compute units x 2 KiB).
// *flops = the FLOPs of the matrix instructions of one launch.
hipError_t launch_matrix_rate(const void* src, void* sink, int mix, int iterations, double* flops, hipStream_t stream)
{
    const int cus = device_cus();
    if (mix == 1) hipLaunchKernelGGL(matrix_rate_kernel<1>, dim3(cus), dim3(512), 0, stream, (const unsigned*)src, (float*)sink, iterations);
    else hipLaunchKernelGGL(matrix_rate_kernel<0>, dim3(cus), dim3(512), 0, stream, (const unsigned*)src, (float*)sink, iterations);
    *flops = (double)cus * 8.0 * (double)iterations * 4.0 * 32768.0;
    return hipGetLastError();
}

// ---- read rate -----------------------------------------------------------------------------------------------------
// Nothing but 16-byte loads of `bytes` bytes, 8 in flight per lane, summed and thrown away: what the memory system
// delivers to a kernel that only reads - the ceiling the split-KV kernels live under, below the nominal HBM figure.
typedef float float4r __attribute__((ext_vector_type(4)));
template <bool NT>
__global__ __launch_bounds__(256) void read_rate_kernel(const float4r* __restrict__ src, float* sink, size_t vecs_per_wg)
{
    const float4r* p = src + (size_t)blockIdx.x * vecs_per_wg + threadIdx.x;
    float4r acc = {0.0f, 0.0f, 0.0f, 0.0f};
    for (size_t i = 0; i < vecs_per_wg; i += 256 * 8) {
        float4r v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = NT ? __builtin_nontemporal_load(p + i + u * 256) : p[i + u * 256];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc += v[u];
    }
    if (acc[0] + acc[1] + acc[2] + acc[3] == 12345.678f) sink[blockIdx.x] = acc[0];      // (never: keeps the loads alive)
}

// bytes: a multiple of 4096 workgroups x 32 KiB; sink: 16 KiB.
hipError_t launch_read_rate(const void* src, void* sink, size_t bytes, int nontemporal, hipStream_t stream)
{
    const int wgs = 4096;
    const size_t vecs_per_wg = bytes / 16 / wgs;
    if (nontemporal) hipLaunchKernelGGL((read_rate_kernel<true>), dim3(wgs), dim3(256), 0, stream, (const float4r*)src, (float*)sink, vecs_per_wg);
    else hipLaunchKernelGGL((read_rate_kernel<false>), dim3(wgs), dim3(256), 0, stream, (const float4r*)src, (float*)sink, vecs_per_wg);
    return hipGetLastError();
}

// Writes `pattern` into every 32-bit word of a 160 KiB LDS allocation, one workgroup per LDS in flight: what the next
// kernels on those compute units find in LDS they have not written themselves.
__global__ __launch_bounds__(256) void lds_fill_kernel(uint32_t* sink, uint32_t pattern)
{
    extern __shared__ uint32_t lds_words[];
    constexpr int kWords = 160 * 1024 / 4;
    for (int i = threadIdx.x; i < kWords; i += 256) lds_words[i] = pattern;
    __syncthreads();
    uint32_t acc = 0;
    for (int i = threadIdx.x; i < kWords; i += 256 * 64) acc ^= lds_words[(i + 4099) % kWords];
    if (acc == 0x9e3779b9u && pattern != 0x9e3779b9u) sink[0] = acc;                      // (never: keeps the stores alive)
}

// sink: 4 bytes.  1024 workgroups: four passes over 256 compute units, so each one's LDS is written whichever way the
// dispatcher spreads them.
hipError_t launch_lds_fill(void* sink, uint32_t pattern, hipStream_t stream)
{
    constexpr int kBytes = 160 * 1024;
    static thread_local int configured_dev = -1;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (configured_dev != dev) {
        e = hipFuncSetAttribute((const void*)lds_fill_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kBytes);
        if (e != hipSuccess) return e;
        configured_dev = dev;
    }
    hipLaunchKernelGGL(lds_fill_kernel, dim3(1024), dim3(256), kBytes, stream, (uint32_t*)sink, pattern);
    return hipGetLastError();
}

}  // namespace incin_rocm
