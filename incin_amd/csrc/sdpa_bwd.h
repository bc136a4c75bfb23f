// Launch parameters of the attention backward kernels (sdpa_bwd_mfma.hip, sdpa_bwd_f32.hip, sdpa_bwd_generic.hip), shared with the C ABI layer.
#pragma once
#include <hip/hip_runtime.h>

#include "sdpa_params.h"

namespace incin_rocm {

struct SdpaBwdParams {
    SdpaParams f;                  // the forward's operands and masks; f.o = the forward's output, f.lse = its normalisers
    const void* d_o;               // upstream gradient, [B, Hq, Sq, D] by strides
    void* d_q;
    void* d_k;
    void* d_v;
    float* neg_l2;                 // workspace, [B, Hq, Sq]: -L_i log2(e) (the normalisers, negated, in log2 units)
    float* neg_delta;              // workspace, [B, Hq, Sq]: -D_i = -(dO_i . O_i)
    int64_t do_sb, do_sh, do_ss;
    int64_t dq_sb, dq_sh, dq_ss;
    int64_t dk_sb, dk_sh, dk_ss;
    int64_t dv_sb, dv_sh, dv_ss;
    // f32 matrix-core kernels on a launch that does not fill the device: the key tiles of a dQ workgroup are dealt to parts_q
    // workgroups, the query tiles of a dK/dV workgroup to parts_kv (1, 2 or 4 each).  Part 0 writes the gradient's rows; part
    // k > 0 writes its sums into plane k - 1 of a contiguous f32 copy of the gradient's shape in the workspace, and a pass
    // after the kernel adds the planes to the rows in order.
    int32_t parts_q, parts_kv;
    float* part_dq;                // workspace, [parts_q - 1][B, Hq, Sq, D]
    float* part_dk;                // workspace, [parts_kv - 1][B, Hkv, Skv, D]
    float* part_dv;                // workspace, [parts_kv - 1][B, Hkv, Skv, Dv]
};

hipError_t launch_sdpa_bwd_mfma(const SdpaBwdParams& bp, int dtype, hipStream_t stream);
hipError_t launch_sdpa_bwd_f32(const SdpaBwdParams& bp, hipStream_t stream);
hipError_t launch_sdpa_bwd_generic(const SdpaBwdParams& bp, int dtype, hipStream_t stream);

}  // namespace incin_rocm
