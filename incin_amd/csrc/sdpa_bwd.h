// Launch parameters of the attention backward kernels (sdpa_bwd_mfma.hip), shared with the C ABI layer.
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
    float* delta;                  // workspace, [B, Hq, Sq]
    int64_t do_sb, do_sh, do_ss;
    int64_t dq_sb, dq_sh, dq_ss;
    int64_t dk_sb, dk_sh, dk_ss;
    int64_t dv_sb, dv_sh, dv_ss;
};

hipError_t launch_sdpa_bwd_mfma(const SdpaBwdParams& bp, int dtype, hipStream_t stream);

}  // namespace incin_rocm
