// Launch parameters of the key/value cache append (kv_append.hip), shared with the C ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace incin_rocm {

struct KvAppendParams {
    const char* k_new;      // [B, Hkv, S_new, D] by strides (elements)
    const char* v_new;      // [B, Hkv, S_new, Dv]
    char* k_cache;          // [B, Hkv, S_max, D]
    char* v_cache;          // [B, Hkv, S_max, Dv]
    int32_t* kv_lens;       // [B]: rows already in the cache
    int64_t kn_sb, kn_sh, kn_ss, vn_sb, vn_sh, vn_ss;
    int64_t kc_sb, kc_sh, kc_ss, vc_sb, vc_sh, vc_ss;
    int32_t B, Hkv, S_new, S_max;
    int32_t k_row_bytes, v_row_bytes, elem;      // bytes of a K row, of a V row, of an element
};

hipError_t launch_kv_append(const KvAppendParams& p, bool vec16, hipStream_t stream);

}  // namespace incin_rocm
