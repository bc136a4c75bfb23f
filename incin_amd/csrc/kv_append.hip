// Appends new key / value rows to a preallocated cache at per-batch positions kept on the device, so that a
// decode step (append the token's K and V, attend over the cache with kv_lens) needs nothing from the host and
// can be recorded once into a launch graph and replayed per token.
//
// Two dispatches, stream-ordered: the copy reads the positions, then a one-workgroup kernel advances them.
#include "kv_append.h"

namespace incin_rocm {

typedef unsigned int uint4v __attribute__((ext_vector_type(4)));

// One workgroup per (batch, head, new row): the K row, then the V row, 16 bytes per lane where the rows allow it.
template <bool VEC16>
__global__ __launch_bounds__(64) void kv_append_kernel(KvAppendParams p)
{
    const int s = blockIdx.x % p.S_new;
    const int h = (blockIdx.x / p.S_new) % p.Hkv;
    const int b = blockIdx.x / (p.S_new * p.Hkv);
    const int64_t pos = (int64_t)p.kv_lens[b] + s;
    if (pos < 0 || pos >= p.S_max) return;            // the cache is full: the row is dropped (see the header)
    const char* ks = p.k_new + (b * p.kn_sb + h * p.kn_sh + s * p.kn_ss) * p.elem;
    const char* vs = p.v_new + (b * p.vn_sb + h * p.vn_sh + s * p.vn_ss) * p.elem;
    char* kd = p.k_cache + (b * p.kc_sb + h * p.kc_sh + pos * p.kc_ss) * p.elem;
    char* vd = p.v_cache + (b * p.vc_sb + h * p.vc_sh + pos * p.vc_ss) * p.elem;
    if (VEC16) {
        for (int i = threadIdx.x * 16; i < p.k_row_bytes; i += 64 * 16) *(uint4v*)(kd + i) = *(const uint4v*)(ks + i);
        for (int i = threadIdx.x * 16; i < p.v_row_bytes; i += 64 * 16) *(uint4v*)(vd + i) = *(const uint4v*)(vs + i);
    } else {
        for (int i = threadIdx.x * p.elem; i < p.k_row_bytes; i += 64 * p.elem)
            for (int e = 0; e < p.elem; ++e) kd[i + e] = ks[i + e];
        for (int i = threadIdx.x * p.elem; i < p.v_row_bytes; i += 64 * p.elem)
            for (int e = 0; e < p.elem; ++e) vd[i + e] = vs[i + e];
    }
}

__global__ __launch_bounds__(64) void kv_advance_kernel(int32_t* kv_lens, int B, int S_new, int S_max)
{
    for (int b = threadIdx.x; b < B; b += 64) {
        const int64_t n = (int64_t)kv_lens[b] + S_new;
        kv_lens[b] = (int32_t)(n > S_max ? S_max : n);
    }
}

hipError_t launch_kv_append(const KvAppendParams& p, bool vec16, hipStream_t stream)
{
    const int64_t rows = (int64_t)p.B * p.Hkv * p.S_new;
    if (rows > 0) {
        if (vec16) hipLaunchKernelGGL(kv_append_kernel<true>, dim3((unsigned)rows), dim3(64), 0, stream, p);
        else hipLaunchKernelGGL(kv_append_kernel<false>, dim3((unsigned)rows), dim3(64), 0, stream, p);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (p.B > 0 && p.S_new > 0) hipLaunchKernelGGL(kv_advance_kernel, dim3(1), dim3(64), 0, stream, p.kv_lens, p.B, p.S_new, p.S_max);
    return hipGetLastError();
}

}  // namespace incin_rocm
