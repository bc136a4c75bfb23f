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
    // Matrix-core kernels on a launch that does not fill the device: the key tiles of a dQ workgroup are dealt to parts_q
    // workgroups (f32 only), the query tiles of a dK/dV workgroup to parts_kv (1, 2, 4; 16-bit storage also 8).  The sums meet in
    // planes of the workspace - contiguous f32 copies of the gradient's shape - and a pass behind the kernel adds them in
    // order.  f32: part 0 writes the gradient's rows itself and part k > 0 plane k - 1, which the pass adds to the rows; 16-bit
    // storage: every part writes a plane, and the pass rounds their sum into the rows.
    int32_t parts_q, parts_kv;
    float* part_dq;                // workspace, f32: [parts_q - 1][B, Hq, Sq, D]
    float* part_dk;                // workspace, f32: [parts_kv - 1][B, Hkv, Skv, D]; 16-bit storage: [parts_kv][...]
    float* part_dv;                // workspace, likewise [..][B, Hkv, Skv, Dv]
};

hipError_t launch_sdpa_bwd_mfma(const SdpaBwdParams& bp, int dtype, hipStream_t stream);
hipError_t launch_sdpa_bwd_f32(const SdpaBwdParams& bp, hipStream_t stream);
hipError_t launch_sdpa_bwd_generic(const SdpaBwdParams& bp, int dtype, hipStream_t stream);

}  // namespace incin_rocm
