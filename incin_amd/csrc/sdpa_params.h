// Kernel-side view of one attention launch (filled from incin_rocm_sdpa_desc_t by
// the host dispatcher after validation).  Strides are in elements.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace incin_rocm {

struct SdpaParams {
    const void* q;
    const void* k;
    const void* v;
    void* o;
    const void* mask;          // nullable dense additive mask (same dtype as q)
    const int32_t* kv_lens;    // nullable, B entries
    const int32_t* q_lens;     // nullable, B entries: query rows at and beyond are padding (output unspecified)
    float* lse;                // nullable, [B, Hq, Sq]: natural-log softmax normaliser of every row (generic and MFMA prefill kernels)
    int64_t q_sb, q_sh, q_ss;
    int64_t k_sb, k_sh, k_ss;
    int64_t v_sb, v_sh, v_ss;
    int64_t o_sb, o_sh, o_ss;
    int64_t m_sb, m_sh, m_si, m_sj;
    int32_t B, Hq, Hkv, G;     // G = Hq / Hkv
    int32_t Sq, Skv, D, Dv;
    int32_t Dp;                // matrix-core kernels: the head dimension their instance is built for (64 or 128); D and Dv fit in it, zero-padded
    float scale;
    int32_t causal;
    int32_t interleave;        // MFMA prefill kernels: (batch, KV head) pairs per group of the work list, set by their launchers
    int32_t deal_groups;       // MFMA prefill kernels: (batch, KV head) pairs are dealt to the 8 XCDs in turn (else: contiguous eighths)
    // split-KV only
    int32_t num_splits;
    int32_t split_len;         // keys per split (multiple of the kernel's key tile)
    float* ws_acc;             // [B, Hq, Sq, num_splits, Dp] f32 partial numerators (Dp == Dv for the vector-ALU kernel)
    float* ws_ml;              // [B, Hq, Sq, num_splits, 2]  running max (natural-log domain) and denominator
    // matrix-core prefill kernels with a dense mask: one byte per block of 32 query rows x 32 keys (0 mixed, 1 all zero,
    // 2 all -inf), written by mask_classify_kernel ahead of the attention kernel, in the caller's workspace;
    // [mask batch entries][mask heads][ceil(Sq / 32)][ceil(Skv / 32)], an extent of 1 where the mask is broadcast
    const uint8_t* mask_flags;
    // and, for the 16-bit prefill kernel, one int per mask row ([mask batch entries][mask heads][Sq, or 1 where the rows are
    // broadcast]): n if the row is n zeros followed by -inf to its end - a causal mask, key padding, both - else -1, written by
    // mask_row_limits_kernel.  A workgroup whose rows all have one needs no mask values, only the limits.  Null: not provided.
    const int32_t* mask_lims;
    int32_t lims_rows;         // rows per block of the launch that takes the blocks whose rows all have a limit (128 or 256; set by the launcher)
    int32_t mask_vec;          // 16-bit MFMA kernel: the mask's rows allow 8-byte loads of 4 consecutive keys
    int32_t mask_chunks;       // 16-bit MFMA prefill kernel: the mask's rows can be copied into LDS 16 bytes (8 keys) at a time
};

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

template <typename T> __device__ __forceinline__ float to_f32(T x) { return (float)x; }
template <typename T> __device__ __forceinline__ T from_f32(float x) { return (T)x; }

// Number of keys a query row may look at, before kv_lens: causal alignment puts
// the last query on the last key (query i sees keys j <= i + Skv - Sq).
__device__ __forceinline__ int causal_limit(int i, int Sq, int Skv) { return i + (Skv - Sq) + 1; }

__device__ __forceinline__ int clampi(int x, int lo, int hi) { return x < lo ? lo : (x > hi ? hi : x); }

// Where the block flags of (batch b, query head hq) start, and the flags per row of blocks.
__device__ __forceinline__ const uint8_t* mask_flags_of(const SdpaParams& p, int b, int hq)
{
    const int nkb = (p.Skv + 31) / 32, nrb = (p.Sq + 31) / 32;
    const int Hm = p.m_sh ? p.Hq : 1;
    const int64_t bh = (int64_t)(p.m_sb ? b : 0) * Hm + (p.m_sh ? hq : 0);
    return p.mask_flags + bh * nrb * nkb;
}

// Where the row limits of (batch b, query head hq) start.
__device__ __forceinline__ const int32_t* mask_lims_of(const SdpaParams& p, int b, int hq)
{
    const int Hm = p.m_sh ? p.Hq : 1;
    const int64_t bh = (int64_t)(p.m_sb ? b : 0) * Hm + (p.m_sh ? hq : 0);
    return p.mask_lims + bh * (p.m_si ? p.Sq : 1);
}

}  // namespace incin_rocm
