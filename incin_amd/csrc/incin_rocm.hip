// Host side of the C ABI declared in include/incin_rocm.h: device table, buffers,
// streams/events, descriptor validation and kernel dispatch.  No kernel lives
// here and no CPU implementation of the operator exists in this library: a
// request no GPU kernel covers is an error, never a host fallback.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "../../include/incin_rocm.h"
#include "copy.h"
#include "kv_append.h"
#include "sdpa_bwd.h"
#include "sdpa_params.h"

namespace incin_rocm {
hipError_t launch_sdpa_generic(const SdpaParams& p, int dtype, hipStream_t stream);
hipError_t launch_sdpa_prefill_mfma(const SdpaParams& p, int dtype, hipStream_t stream);
hipError_t launch_matrix_rate(const void* src, void* sink, int mix, int iterations, double* flops, hipStream_t stream);
hipError_t launch_sdpa_prefill_f32(const SdpaParams& p, hipStream_t stream);
hipError_t launch_sdpa_prefill_wide(const SdpaParams& p, int dtype, hipStream_t stream);
hipError_t launch_mask_classify(const SdpaParams& p, int dtype, hipStream_t stream);
hipError_t launch_mask_row_limits(const void* mask, int dtype, const int64_t shape[4], const int64_t strides[4], int32_t* lims, hipStream_t stream);
hipError_t launch_sdpa_decode_f32_limits(const SdpaParams& p, hipStream_t stream);
hipError_t launch_sdpa_decode(const SdpaParams& p, int dtype, hipStream_t stream);
hipError_t launch_sdpa_decode_mfma(const SdpaParams& p, int dtype, hipStream_t stream);
hipError_t launch_read_rate(const void* src, void* sink, size_t bytes, int nontemporal, hipStream_t stream);
hipError_t launch_lds_fill(void* sink, uint32_t pattern, hipStream_t stream);
int decode_mfma_chunk_rows(int R, int dtype, int d_pad);
int decode_mfma_workgroups_per_cu(int chunk_rows, int64_t split_len, int dtype, int d_pad);
int decode_keys_per_tile(int dtype, int D, int R);
}  // namespace incin_rocm

using incin_rocm::SdpaParams;

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_fail(hipError_t e, const char* what)
{
    int code = (e == hipErrorOutOfMemory) ? INCIN_ROCM_ENOMEM
             : (e == hipErrorInvalidDevice || e == hipErrorNoDevice) ? INCIN_ROCM_EDEVICE
                                                                     : INCIN_ROCM_ERUNTIME;
    return fail(code, "ROCm %s failed: %s (%s)", what, hipGetErrorString(e), hipGetErrorName(e));
}

#define HIP_TRY(expr, what)                         \
    do {                                            \
        hipError_t _e = (expr);                     \
        if (_e != hipSuccess) return hip_fail(_e, what); \
    } while (0)

int use_device(int32_t dev)
{
    // the device count does not change while the process lives: asked once; the current device is only switched when
    // it is another one (both calls are per-thread state lookups, no driver round trip on the launch path)
    static std::atomic<int> count{-1};
    int n = count.load(std::memory_order_relaxed);
    if (n < 0) {
        hipError_t e = hipGetDeviceCount(&n);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return fail(INCIN_ROCM_EDEVICE, "ROCm device query failed: %s", hipGetErrorString(e));
        }
        count.store(n, std::memory_order_relaxed);
    }
    if (dev < 0 || dev >= n) return fail(INCIN_ROCM_EDEVICE, "invalid ROCm device ordinal %d (%d device(s) present)", dev, n);
    int cur = -1;
    if (hipGetDevice(&cur) != hipSuccess || cur != dev) HIP_TRY(hipSetDevice(dev), "hipSetDevice");
    return 0;
}

size_t dtype_size(int dtype) { return dtype == INCIN_ROCM_F32 ? 4 : 2; }


// Compute units of device `dev` (256 when it cannot be asked, e.g. a workspace query on a machine without a device:
// only launch geometry depends on it).
int compute_units_of(int dev)
{
    static std::atomic<int> cached[64];
    if (dev < 0 || dev >= 64) return 256;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            n = 256;
        }
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// What the dispatcher decided for one descriptor.
struct Plan {
    int impl;
    int splits;
    int split_len;
    size_t ws_bytes;
    size_t lims_offset;      // dense mask on the prefill kernels: where the mask's row limits start in the workspace (0: none)
    bool lims_splitkv;       // f32 with a dense mask: the blocks whose rows all have a limit go through the f32 split-KV kernel first
    bool empty;      // nothing to compute
};

bool fast_layout_ok(const incin_rocm_sdpa_desc_t* d, int vec)
{
    // 16-byte vector loads of whole rows: row starts and strides must be multiples of the vector.
    if (!aligned16(d->q) || !aligned16(d->k) || !aligned16(d->v) || !aligned16(d->o)) return false;
    for (int a = 0; a < 3; ++a) {
        if (d->q_stride[a] % vec || d->k_stride[a] % vec || d->v_stride[a] % vec || d->o_stride[a] % vec) return false;
    }
    return true;
}

// The rows of a 16-bit dense mask can be read four keys (8 bytes) at a time: unit stride along the keys, every row 8-byte aligned.
bool mask_rows_vector_loadable(const incin_rocm_sdpa_desc_t* d)
{
    return d->add_mask && d->mask_stride[3] == 1 && (reinterpret_cast<uintptr_t>(d->add_mask) & 7u) == 0 &&
           d->mask_stride[0] % 4 == 0 && d->mask_stride[1] % 4 == 0 && d->mask_stride[2] % 4 == 0;
}

// A 16-bit dense mask the matrix-core split-KV kernel can copy into LDS 16 bytes (8 keys) at a time: unit key stride, a key
// count that is a multiple of 8, every row 16-byte aligned, non-negative strides, and offsets inside a batch entry that fit
// the 32-bit offsets of its copies.
bool mask_rows_chunk_copyable(const incin_rocm_sdpa_desc_t* d)
{
    if (!d->add_mask || d->mask_stride[3] != 1 || d->Skv % 8 != 0 || (reinterpret_cast<uintptr_t>(d->add_mask) & 15u) != 0) return false;
    for (int a = 0; a < 3; ++a)
        if (d->mask_stride[a] < 0 || d->mask_stride[a] % 8 != 0) return false;
    const int64_t extent = (d->Hq - 1) * d->mask_stride[1] + (d->Sq - 1) * d->mask_stride[2] + d->Skv;
    return extent < (1LL << 29);
}

// A 16-bit dense mask whose values the prefill kernel can bring into LDS by 16-byte copies, 32 rows x 64 keys at a time from a
// descriptor that starts at the first of the 32 rows: unit key stride, a key count that is a multiple of 8 (no copy straddles
// the end of the last row), every row 16-byte aligned, non-negative strides, 32 rows within the copies' 32-bit offsets.
bool mask_rows_stageable(const incin_rocm_sdpa_desc_t* d)
{
    if (!d->add_mask || d->mask_stride[3] != 1 || d->Skv % 8 != 0 || (reinterpret_cast<uintptr_t>(d->add_mask) & 15u) != 0) return false;
    for (int a = 0; a < 3; ++a)
        if (d->mask_stride[a] < 0 || d->mask_stride[a] % 8 != 0) return false;
    return (32 * d->mask_stride[2] + d->Skv) < (1LL << 29);
}

int make_plan(const incin_rocm_sdpa_desc_t* d, Plan* plan)
{
    if (!d) return fail(INCIN_ROCM_EINVAL, "scaled_dot_product_attention: null descriptor");
    if (d->dtype != INCIN_ROCM_F32 && d->dtype != INCIN_ROCM_F16 && d->dtype != INCIN_ROCM_BF16)
        return fail(INCIN_ROCM_EDTYPE, "scaled_dot_product_attention: unsupported dtype tag %d on backend Rocm (f32, f16, bf16 only)", d->dtype);
    const int64_t lim = 0x7fffffffLL;
    if (d->B < 0 || d->Hq < 0 || d->Hkv < 0 || d->Sq < 0 || d->Skv < 0 || d->D < 0 || d->Dv < 0)
        return fail(INCIN_ROCM_ESHAPE, "scaled_dot_product_attention: negative extent");
    if (d->B > lim || d->Hq > lim || d->Hkv > lim || d->Sq > lim || d->Skv > lim || d->D > lim || d->Dv > lim)
        return fail(INCIN_ROCM_ESHAPE, "scaled_dot_product_attention: extent exceeds 2^31-1");
    plan->impl = INCIN_ROCM_IMPL_GENERIC;
    plan->splits = 1;
    plan->split_len = (int)d->Skv;
    plan->ws_bytes = 0;
    plan->lims_offset = 0;
    plan->lims_splitkv = false;
    plan->empty = (d->B == 0 || d->Hq == 0 || d->Sq == 0 || d->Dv == 0);
    if (plan->empty) return 0;
    if (d->Hkv <= 0 || d->Hq % d->Hkv != 0)
        return fail(INCIN_ROCM_ESHAPE,
                    "scaled_dot_product_attention: %lld query heads cannot share %lld key/value heads (batch axes do not broadcast)",
                    (long long)d->Hq, (long long)d->Hkv);
    if (d->B > 65535 || d->Hq > 65535)
        return fail(INCIN_ROCM_ESHAPE, "scaled_dot_product_attention: batch and head counts are limited to 65535 per launch");
    if (!d->q || !d->o || (d->Skv > 0 && (!d->k || !d->v)))
        return fail(INCIN_ROCM_EINVAL, "scaled_dot_product_attention: null tensor pointer");
    if (d->impl < INCIN_ROCM_IMPL_AUTO || d->impl > INCIN_ROCM_IMPL_SPLITKV_MFMA)
        return fail(INCIN_ROCM_EINVAL, "scaled_dot_product_attention: unknown impl %d", d->impl);
    if (d->num_splits < 0) return fail(INCIN_ROCM_EINVAL, "scaled_dot_product_attention: negative num_splits");

    const int vec = d->dtype == INCIN_ROCM_F32 ? 4 : 8;
    const int64_t R = (d->Hq / d->Hkv) * d->Sq;
    // The matrix-core kernels are built for head dimensions 64 and 128; smaller ones (D and Dv need not be equal) run in
    // the instance that holds them, padded with zeros on the way into LDS, as long as rows stay whole 16-byte vectors.
    // Above 128 (up to 256): an instance for 256 of the split-KV kernels (16-bit and f32, any number of query positions) and of
    // the 16-bit prefill kernel (sdpa_prefill_wide.hip, no dense mask).  The vector-ALU split-KV kernel takes D == Dv in
    // {64, 128} as they are.
    const int64_t d_max = std::max(d->D, d->Dv);
    const int64_t d_pad = d_max <= 64 ? 64 : d_max <= 128 ? 128 : 256;
    const bool wide = d_pad == 256;
    const bool head_pad_ok = d->D > 0 && d_max <= 256 && d->D % vec == 0 && d->Dv % vec == 0;
    const bool head_exact = d->D == d->Dv && d->D == d_pad && !wide;
    const bool layout_ok = head_pad_ok && fast_layout_ok(d, vec) && d->Skv > 0;
    const bool fast_ok = layout_ok && !d->add_mask;
    // the MFMA kernels address a K/V tile with 32-bit byte offsets from the tile's first row
    const int64_t stride_lim = d->dtype == INCIN_ROCM_F32 ? (1 << 22) : (1 << 24);
    const bool tile_off_ok = d->k_stride[2] >= 0 && d->v_stride[2] >= 0 && d->k_stride[2] < stride_lim && d->v_stride[2] < stride_lim;
    // f32: the IEEE-f32 matrix-core kernel, any finite scale; f16 / bf16: the 16-bit kernels fold the scale into Q in
    // a way that needs it positive.  Both take a dense additive mask (any strides); the 64-row kernel does not.
    // (above 128: sdpa_prefill_wide.hip - 16-bit storage, any finite scale, a dense mask whose rows it can read 8 bytes at a time)
    const bool mfma_ok = wide ? layout_ok && d->dtype != INCIN_ROCM_F32 && tile_off_ok && std::isfinite(d->scale) && (!d->add_mask || mask_rows_vector_loadable(d))
                              : layout_ok && tile_off_ok && std::isfinite(d->scale) && (d->dtype == INCIN_ROCM_F32 || d->scale > 0.0f);
    const bool split_ok = layout_ok && head_exact && d->Sq <= 64;      // (the vector-ALU kernel takes a dense mask)
    // the matrix-core split-KV kernels (16-bit and f32): blocks addressed like the prefill kernels' tiles; the f32 kernel and
    // the 256 instances take any number of query positions
    // (the 16-bit kernel also takes a dense mask it can copy into LDS eight keys at a time - not in the form of 64 rows per
    // workgroup at D = 64, where the mask's buffers do not fit beside the rings)
    const bool split_mask_ok = !d->add_mask || (d->dtype != INCIN_ROCM_F32 && mask_rows_chunk_copyable(d) && !(d_pad == 64 && R > 32));
    const bool split_mfma_ok = layout_ok && split_mask_ok && (d->Sq <= 64 || wide || d->dtype == INCIN_ROCM_F32) && tile_off_ok && std::isfinite(d->scale);

    int impl = d->impl;
    if (impl == INCIN_ROCM_IMPL_AUTO) {
        // Few rows per KV head (query heads of the group x query positions) over a long cache: split-KV.  With more
        // than a row or two the vector-ALU kernel runs out of arithmetic before it runs out of bandwidth (measured on
        // 32 x 8 KV heads x 8192 keys: 83 / 82 / 77 / 76 / 54 % of the memory bandwidth at 1 / 2 / 3 / 4 / 5 rows, the
        // matrix-core kernel 86 - 87 % at each); over the shortest caches the matrix-core kernel's one or two workgroups
        // per compute unit have too little to stream, and the vector-ALU kernel keeps those (the thresholds are where
        // the two cross on launches of 268 MB of cache).  With one row per KV head the two kernels are within a few per
        // cent of each other everywhere; the matrix-core one is ahead on launches that run long enough for its longer
        // start-up not to show (3 - 4 % from 1 GB of cache on, behind by 4 - 9 % at 64 - 268 MB).
        // Up to 64 rows the matrix-core kernel reads the cache once; beyond (it would read it once per 64 rows) the
        // prefill kernel takes over, which splits the keys itself when its launch is small (measured level or ahead from
        // 128 rows per KV head on).
        const int64_t esize = (int64_t)dtype_size(d->dtype);
        const int64_t kv_bytes = 2 * d->B * d->Hkv * d->Skv * d->D * esize;
        const int64_t len128 = d->Skv * d_pad * esize / 256;     // cache length in keys of 256 bytes (what the thresholds were measured in)
        // Head dimensions above 128: the 16-bit prefill kernel for 256 where there are more than 64 query positions (128 rows
        // share a K / V tile there, 32 in the split-KV kernel: D = 256 causal prefill 775 - 890 against 340 - 460 TFLOP/s), the
        // split-KV kernels' 256 instance for decode shapes and - f32 has no such prefill kernel - for every f32 shape.
        // That prefill kernel does not split the keys: a launch that gives it workgroups for at most half the compute units
        // (the chunks of a long prompt, few heads) goes 32 rows per workgroup, keys split as needed, through the split-KV
        // kernel (measured, bf16 causal, D = 256: 8 heads x 128 x 8192 0.305 -> 0.039 ms; 32 x 256 x 16384 0.60 -> 0.26;
        // 8 x 1024 x 32768 1.18 -> 0.56; 16 x 1024 x 4096 - 128 workgroups - 0.158 -> 0.121; at 256 workgroups
        // (2 x 32 x 512 x 512) the prefill kernel is ahead, 0.031 against 0.057).
        // Swept over 4 - 32 heads x 128 - 2048 rows x 1024 - 16384 keys (causal, one sequence): the split-KV kernel is ahead
        // (to 0.06 of the prefill kernel's time) up to a quarter of the compute units' worth of 128-row workgroups, and up to
        // half where its 32-row chunks come in whole rounds of the compute units (its workgroups then finish together);
        // with a ragged last round (192, 288, 384 chunks) it is 1.1 - 1.5 times behind from 48 - 72 workgroups on, and over
        // fewer than 2048 keys a ragged round is all there is.
        const int64_t cus_w = compute_units_of(d->device);
        const int64_t wgs_w = d->B * d->Hq * ((d->Sq + 127) / 128), chunks_w = d->B * d->Hkv * ((R + 31) / 32);
        const bool wide_underfilled = (wgs_w * 4 <= cus_w && (d->Skv >= 2048 || chunks_w * 2 <= cus_w || chunks_w % cus_w == 0)) ||
                                      (wgs_w * 2 <= cus_w && chunks_w % cus_w == 0);
        // The prefill kernel for 256 splits the keys like the one for 128 (a launch of at most one workgroup per compute unit over
        // 4096 keys or more, four times the rows: see below); where those splits give every compute unit a workgroup it is well
        // ahead of the split-KV kernel's 32 rows per pass over K and V (32 / 8 heads x 256 x 16384 0.257 -> 0.153 ms; 8 / 2 heads x
        // 1024 x 32768 0.57 -> 0.27; 64 / 8 heads x 128 x 32768 0.59 -> 0.29; 16 heads x 1024 x 4096 0.138 -> 0.096), and behind
        // where they do not (8 heads x 128 x 8192: 64 workgroups, 0.053 against 0.036).
        const int64_t wide_splits = (wgs_w <= cus_w && d->Skv >= 4096 && d->Skv >= 4 * d->Sq && !d->q_lens && d->num_splits == 0)
                                        ? std::min<int64_t>(2 * cus_w / wgs_w, d->Skv / 1024) : (d->num_splits > 1 ? d->num_splits : 1);
        const bool wide_split_fills = wide_splits > 1 && wgs_w * wide_splits >= cus_w && !d->add_mask && d->dtype != INCIN_ROCM_F32;
        // (with a dense mask the prefill kernel keeps launches of more than 64 positions: its block flags skip what the mask hides)
        if (wide && mfma_ok && d->Sq > 64 && (wide_split_fills || !(split_mfma_ok && wide_underfilled && !d->add_mask))) impl = INCIN_ROCM_IMPL_MFMA;
        else if (wide && split_mfma_ok) impl = INCIN_ROCM_IMPL_SPLITKV_MFMA;
        // f32 (sdpa_decode_f32.hip): from two rows per KV head on, whatever the count - the f32 prefill kernel would spend a
        // 32-row matrix instruction on every query head's few rows (32 heads of a group at one position each: 8.4 ms
        // against 0.23), and where it packs as well (64 positions of one head) the split-KV form is still ahead (0.22
        // against 0.28 ms on 8 x 8 heads x 8192 keys); the vector-ALU kernel is level at 2 rows and behind from 4 on
        // (4 rows, 268 MB of cache: 5.6 against 4.8 TB/s; 8 rows: 6.6 against 3.4).  That holds over short caches too since the
        // 32-row form runs two workgroups per compute unit (48 positions x 16 heads x 16 sequences of 300 keys: 0.020 against
        // the prefill kernel's 0.030 ms).
        // One row per KV head (swept over 1 - 32 sequences x 8 - 32 heads x 512 - 16384 keys): the matrix-core kernel is level
        // from 500 MB of cache on and up to 2.8 times ahead below (its splits fill the device where the vector-ALU kernel's
        // do not), except over the shortest caches at D = 64 (512 keys: 1.1 - 1.4 times behind).
        else if (d->dtype == INCIN_ROCM_F32 && split_mfma_ok && d->Sq <= 64 && len128 >= 256 &&
                 (R >= 2 || d->Skv >= (d_pad == 64 ? 1024 : 512)))
            impl = INCIN_ROCM_IMPL_SPLITKV_MFMA;
        // f32 prefill launches that give the prefill kernel at most two 128-row workgroups per compute unit (one round of what a
        // compute unit holds; since the 32-row form runs two workgroups per compute unit, longest chunks first: 2 x 16 heads x
        // 2048 x 2048 at D = 128, 512 workgroups' worth, 0.384 -> 0.316 ms; 4 x 16 x 1024 x 1024 0.197 -> 0.180; level at 640
        // workgroups' worth at D = 64; the prefill kernel 1.1 - 1.3 times ahead from 1024 on): the split-KV kernel
        // takes them 32 rows per workgroup with the keys dealt to its four wavefronts - four times the workgroups, a quarter
        // of the keys per wavefront - where the prefill kernel's wavefronts each walk all keys for their 32 rows behind
        // 64-cycle matrix instructions (measured, causal: one head of 128 x 128 13.3 -> 8.6 us; 2 x 8 heads x 512 x 512 at
        // D = 128 73 -> 28; 128 workgroups' worth of 1024 x 1024 80 -> 33; 256 - 4 x 8 heads x 1024 x 1024 at D = 64 - 80 -> 65; level at 512).
        // Not the chunks of a long prompt, where the prefill kernel splits the keys itself (below) and runs at 80 % of the peak.
        else if (d->dtype == INCIN_ROCM_F32 && split_mfma_ok && d->Sq > 64 && !(d->Skv >= 4096 && d->Skv >= 4 * d->Sq) &&
                 d->B * d->Hq * ((d->Sq + 127) / 128) <= 2 * compute_units_of(d->device))
            impl = INCIN_ROCM_IMPL_SPLITKV_MFMA;
        // f16 / bf16 (sdpa_decode_mfma.hip): the thresholds described above
        else if (d->dtype != INCIN_ROCM_F32 && split_mfma_ok && len128 >= 256 &&
            ((R == 1 && len128 >= 1024 && kv_bytes >= (512LL << 20)) || (R >= 2 && R <= 3 && len128 >= 512) || (R >= 4 && R <= 64)))
            impl = INCIN_ROCM_IMPL_SPLITKV_MFMA;
        else if (split_ok && R <= 8 && d->Skv >= 256) impl = INCIN_ROCM_IMPL_SPLITKV;
        // a head dimension that is padded into its instance has no vector-ALU kernel: one row per KV head, too, goes through
        // the matrix-core split-KV kernels
        else if (!head_exact && split_mfma_ok && d->Sq <= 64 && len128 >= 256 && (d->dtype == INCIN_ROCM_F32 || R <= 64)) impl = INCIN_ROCM_IMPL_SPLITKV_MFMA;
        else if (mfma_ok) impl = INCIN_ROCM_IMPL_MFMA;
        else if (split_ok && R <= 8) impl = INCIN_ROCM_IMPL_SPLITKV;
        else impl = INCIN_ROCM_IMPL_GENERIC;
    }
    if (impl == INCIN_ROCM_IMPL_MFMA && !mfma_ok)
        return fail(INCIN_ROCM_EUNSUPPORTED,
                    "scaled_dot_product_attention: the MFMA prefill kernels need D and Dv <= 128 (f16/bf16: 256) in whole 16-byte vectors and 16-byte aligned rows; for f16/bf16 up to 128 also scale > 0");
    if (impl == INCIN_ROCM_IMPL_MFMA64)
        return fail(INCIN_ROCM_EUNSUPPORTED,
                    "scaled_dot_product_attention: the 64-row MFMA prefill kernel has been retired (INCIN_ROCM_IMPL_MFMA covers its shapes)");
    if (impl == INCIN_ROCM_IMPL_SPLITKV_MFMA && !split_mfma_ok)
        return fail(INCIN_ROCM_EUNSUPPORTED,
                    "scaled_dot_product_attention: the matrix-core split-KV kernels need D and Dv <= 256 in whole 16-byte vectors, Sq <= 64 (any Sq in f32 and above 128), no dense mask in f32 (16-bit: one with unit key stride, 16-byte aligned rows and a key count that is a multiple of 8; at D = 64 up to 32 rows per KV head), a finite scale and 16-byte aligned rows");
    if (impl == INCIN_ROCM_IMPL_SPLITKV && !split_ok)
        return fail(INCIN_ROCM_EUNSUPPORTED,
                    "scaled_dot_product_attention: the split-KV kernel needs D == Dv in {64,128}, Sq <= 64 and 16-byte aligned rows");
    if (impl == INCIN_ROCM_IMPL_GENERIC && (d->D > 256 || d->Dv > 256))
        return fail(INCIN_ROCM_EUNSUPPORTED,
                    "scaled_dot_product_attention: head dimension %lld/%lld exceeds 256, no Rocm kernel covers it",
                    (long long)d->D, (long long)d->Dv);
    plan->impl = impl;

    if (impl == INCIN_ROCM_IMPL_SPLITKV) {
        const int rmax = R <= 1 ? 1 : R <= 2 ? 2 : R <= 4 ? 4 : 8;
        const int64_t nchunks = (R + rmax - 1) / rmax;
        const int tile = 4 * incin_rocm::decode_keys_per_tile(d->dtype, (int)d->D, (int)(R > 8 ? 8 : R));
        int64_t splits = d->num_splits;
        if (splits == 0) {
            // enough workgroups for ~8 per compute unit, each split at least 512 keys
            const int64_t groups = d->B * d->Hkv * nchunks;
            splits = (2048 + groups - 1) / groups;
            const int64_t max_by_len = d->Skv / 512 > 0 ? d->Skv / 512 : 1;
            if (splits > max_by_len) splits = max_by_len;
            if (splits < 1) splits = 1;
        }
        int64_t split_len = (d->Skv + splits - 1) / splits;
        split_len = (split_len + tile - 1) / tile * tile;
        splits = (d->Skv + split_len - 1) / split_len;
        if (splits > 65535) return fail(INCIN_ROCM_ESHAPE, "scaled_dot_product_attention: too many splits");
        if (d->Hkv * nchunks > 65535) return fail(INCIN_ROCM_ESHAPE, "scaled_dot_product_attention: too many head groups for one launch");
        plan->splits = (int)splits;
        plan->split_len = (int)split_len;
        plan->ws_bytes = splits > 1 ? (size_t)(d->B * d->Hq * d->Sq * splits) * (size_t)(d_pad + 2) * sizeof(float) : 0;
    }
    if (impl == INCIN_ROCM_IMPL_SPLITKV_MFMA) {
        // One workgroup per (batch, KV head, chunk of 32 or 64 rows, split).  A compute unit holds one at a time (its LDS
        // is the ring of blocks in flight) - two when the splits are short enough for the two-slot rings - so the
        // workgroups of a launch, all of equal length, run in rounds.  Take the number of splits that leaves the last
        // round fullest, among those that keep at least 256 keys per split, preferring fewer splits at (nearly) equal
        // filling: fewer partial results to combine.
        const int64_t chunk = incin_rocm::decode_mfma_chunk_rows((int)std::min<int64_t>(R, 1 << 20), d->dtype, (int)d_pad);
        const int64_t nchunks = (R + chunk - 1) / chunk;
        const int64_t groups = d->B * d->Hkv * nchunks;
        int64_t splits = d->num_splits;
        if (splits == 0) {
            const int64_t cus = compute_units_of(d->device);
            // (from 65536 keys on a split keeps at least 1024: with one or two groups the filling alone would ask for 512 splits of
            //  256 keys, each hardly past its ring's start-up, and a combine pass over 512 partial results per row - one sequence
            //  of 131072 keys on one KV head: 35.9 us in 512 splits, 26.5 in 256, 24.1 in 128, 30.6 in 64)
            const int64_t min_len = d->Skv >= 65536 ? 1024 : 256;
            const int64_t max_by_len = d->Skv / min_len > 0 ? d->Skv / min_len : 1;
            const int64_t max_splits = std::min<int64_t>(max_by_len, std::max<int64_t>(1, 4 * cus / groups));
            auto fill = [&](int64_t s) {           // (with the split length, and so the count, s really leads to)
                const int64_t len = ((d->Skv + s - 1) / s + 255) / 256 * 256;
                const int64_t at_a_time = cus * incin_rocm::decode_mfma_workgroups_per_cu((int)chunk, len, d->dtype, (int)d_pad);
                const int64_t wgs = groups * ((d->Skv + len - 1) / len), rounds = (wgs + at_a_time - 1) / at_a_time;
                return (double)wgs / (double)(rounds * at_a_time);
            };
            double best = 0.0;
            for (int64_t s = 1; s <= max_splits; ++s) best = std::max(best, fill(s));
            splits = 1;
            while (splits < max_splits && fill(splits) < 0.98 * best) ++splits;
        }
        int64_t split_len = (d->Skv + splits - 1) / splits;
        split_len = (split_len + 255) / 256 * 256;      // whole rounds of the four wavefronts' blocks of 32 (D = 128) or 64 keys
        splits = (d->Skv + split_len - 1) / split_len;
        if (splits > 65535) return fail(INCIN_ROCM_ESHAPE, "scaled_dot_product_attention: too many splits");
        if (d->Hkv * nchunks > 65535) return fail(INCIN_ROCM_ESHAPE, "scaled_dot_product_attention: too many head groups for one launch");
        plan->splits = (int)splits;
        plan->split_len = (int)split_len;
        plan->ws_bytes = splits > 1 ? (size_t)(d->B * d->Hq * d->Sq * splits) * (size_t)(d_pad + 2) * sizeof(float) : 0;
    }
    if (impl == INCIN_ROCM_IMPL_MFMA && !d->add_mask && !d->q_lens && !(wide && d->dtype == INCIN_ROCM_F32)) {
        // The prefill kernels (16-bit and f32) run one workgroup per (batch, query head, 128 rows) and a compute unit holds two:
        // when a launch has at most one per compute unit and a long key axis - a chunk of a long prompt, a single
        // sequence - the keys are split as for decode, as many ways as fill the device (1024 keys per split at least:
        // measured best on 32 heads x 128 rows x 8192 keys, 8 splits 32 us against 40 with 4 and 35 with 16), and the
        // splits' partial results go through the split-KV kernels' combine pass.  Only where the key axis is the long one
        // (four times the rows or more): the partial results are rows x splits x D floats, and on a square causal launch
        // writing and combining them costs what the splits gain (one sequence, 8 heads, 4096 x 4096: 61 us whole, 64 in
        // two splits, 74 in four).  num_splits > 0 in the descriptor forces a count.
        const int64_t cus = compute_units_of(d->device);
        const int64_t wgs = d->B * d->Hq * ((d->Sq + 127) / 128);
        int64_t splits = d->num_splits;
        if (splits == 0) {
            splits = 1;
            if (wgs <= cus && d->Skv >= 4096 && d->Skv >= 4 * d->Sq) splits = std::min<int64_t>(2 * cus / wgs, d->Skv / 1024);
        }
        if (splits > 1) {
            int64_t split_len = (d->Skv + splits - 1) / splits;
            split_len = (split_len + 127) / 128 * 128;       // whole pairs of 64-key tiles: every split starts on an even tile
            splits = (d->Skv + split_len - 1) / split_len;
            if (splits > 65535) return fail(INCIN_ROCM_ESHAPE, "scaled_dot_product_attention: too many splits");
            if (splits > 1) {
                plan->splits = (int)splits;
                plan->split_len = (int)split_len;
                plan->ws_bytes = (size_t)(d->B * d->Hq * d->Sq * splits) * (size_t)(d_pad + 2) * sizeof(float);
            }
        }
    }
    if (impl == INCIN_ROCM_IMPL_MFMA && d->add_mask) {
        // one flag per block of 32 query rows x 32 keys of the mask, per mask batch entry and head
        const int64_t nbh = (d->mask_stride[0] ? d->B : 1) * (d->mask_stride[1] ? d->Hq : 1);
        if (nbh > 65535 || (d->Sq + 31) / 32 > 65535)
            return fail(INCIN_ROCM_ESHAPE, "scaled_dot_product_attention: mask too large for one launch of the matrix-core kernels");
        plan->ws_bytes = (size_t)(nbh * ((d->Sq + 31) / 32) * ((d->Skv + 31) / 32) + 255) / 256 * 256;
        // f32: a small launch (what AUTO would hand the f32 split-KV kernel if there were no mask tensor: at most two 128-row
        // blocks per compute unit) whose chunks of 32 rows do not straddle query heads gets the blocks whose mask rows all have
        // a limit computed by that kernel, from the limits, ahead of the prefill kernel's dense-mask launch for the rest
        // (benchmark config 2 with the causal mask as a tensor: 90 -> 66 us)
        plan->lims_splitkv = d->dtype == INCIN_ROCM_F32 && !wide && d->impl == INCIN_ROCM_IMPL_AUTO && !d->q_lens && d->Sq > 64 &&
                             (d->Hq == d->Hkv || d->Sq % 128 == 0) && d->B * d->Hq * ((d->Sq + 127) / 128) <= 2 * compute_units_of(d->device);
        if (d->dtype != INCIN_ROCM_F32 || plan->lims_splitkv) {      // one int per mask row: its limit, if it is zeros up to one and -inf beyond
            plan->lims_offset = plan->ws_bytes;
            plan->ws_bytes += (size_t)(nbh * (d->mask_stride[2] ? d->Sq : 1) * 4 + 255) / 256 * 256;
        }
    }
    return 0;
}

void fill_params(const incin_rocm_sdpa_desc_t* d, const Plan& plan, SdpaParams* p)
{
    memset(p, 0, sizeof(*p));
    p->q = d->q; p->k = d->k; p->v = d->v; p->o = d->o;
    p->mask = d->add_mask;
    p->kv_lens = d->kv_lens;
    p->q_lens = d->q_lens;
    p->lse = d->lse;
    p->q_sb = d->q_stride[0]; p->q_sh = d->q_stride[1]; p->q_ss = d->q_stride[2];
    p->k_sb = d->k_stride[0]; p->k_sh = d->k_stride[1]; p->k_ss = d->k_stride[2];
    p->v_sb = d->v_stride[0]; p->v_sh = d->v_stride[1]; p->v_ss = d->v_stride[2];
    p->o_sb = d->o_stride[0]; p->o_sh = d->o_stride[1]; p->o_ss = d->o_stride[2];
    p->m_sb = d->mask_stride[0]; p->m_sh = d->mask_stride[1]; p->m_si = d->mask_stride[2]; p->m_sj = d->mask_stride[3];
    p->mask_vec = mask_rows_vector_loadable(d);
    p->mask_chunks = d->dtype != INCIN_ROCM_F32 && mask_rows_stageable(d);
    p->B = (int)d->B; p->Hq = (int)d->Hq; p->Hkv = (int)d->Hkv; p->G = (int)(d->Hq / d->Hkv);
    p->Sq = (int)d->Sq; p->Skv = (int)d->Skv; p->D = (int)d->D; p->Dv = (int)d->Dv;
    p->Dp = std::max(d->D, d->Dv) <= 64 ? 64 : std::max(d->D, d->Dv) <= 128 ? 128 : 256;      // (means something to the matrix-core and split-KV kernels only)
    p->scale = d->scale;
    p->causal = d->causal ? 1 : 0;
    p->interleave = 1;
    p->deal_groups = 0;
    p->num_splits = plan.splits;
    p->split_len = plan.split_len;
    if (plan.impl == INCIN_ROCM_IMPL_MFMA) p->mask_flags = d->add_mask ? (const uint8_t*)d->workspace : nullptr;
    if (plan.impl == INCIN_ROCM_IMPL_MFMA && d->add_mask && plan.lims_offset) p->mask_lims = (const int32_t*)((const char*)d->workspace + plan.lims_offset);
    if (!(plan.impl == INCIN_ROCM_IMPL_MFMA && d->add_mask)) p->ws_acc = (float*)d->workspace;
    if (plan.splits > 1) {
        const size_t rows = (size_t)(d->B * d->Hq * d->Sq * plan.splits);
        p->ws_ml = (float*)d->workspace + rows * (size_t)p->Dp;      // partial rows are as wide as the kernel instance
    }
}

}  // namespace

extern "C" {

const char* incin_rocm_last_error(void) { return g_err; }
int incin_rocm_abi_version(void) { return INCIN_ROCM_ABI_VERSION; }
size_t incin_rocm_sizeof_sdpa_desc(void) { return sizeof(incin_rocm_sdpa_desc_t); }
size_t incin_rocm_sizeof_device_info(void) { return sizeof(incin_rocm_device_info_t); }

int incin_rocm_device_count(int32_t* out)
{
    if (!out) return fail(INCIN_ROCM_EINVAL, "device_count: null output");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e == hipErrorNoDevice) {
        (void)hipGetLastError();
        n = 0;
    } else if (e != hipSuccess) {
        (void)hipGetLastError();
        *out = 0;
        return hip_fail(e, "hipGetDeviceCount");
    }
    *out = n;
    return 0;
}

int incin_rocm_device_info(int32_t dev, incin_rocm_device_info_t* out)
{
    if (!out) return fail(INCIN_ROCM_EINVAL, "device_info: null output");
    if (int rc = use_device(dev)) return rc;
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, dev), "hipGetDeviceProperties");
    memset(out, 0, sizeof(*out));
    snprintf(out->name, sizeof(out->name), "%s", prop.name);
    snprintf(out->arch, sizeof(out->arch), "%s", prop.gcnArchName);
    out->compute_units = prop.multiProcessorCount;
    out->clock_khz = prop.clockRate;
    out->memory_clock_khz = prop.memoryClockRate;
    out->memory_bus_bits = prop.memoryBusWidth;
    out->lds_bytes_per_block = (int32_t)prop.sharedMemPerBlock;
    out->wavefront_size = prop.warpSize;
    out->hbm_bytes = (uint64_t)prop.totalGlobalMem;
    return 0;
}

int incin_rocm_alloc(int32_t dev, size_t bytes, void** out)
{
    if (!out) return fail(INCIN_ROCM_EINVAL, "alloc: null output");
    *out = nullptr;
    if (int rc = use_device(dev)) return rc;
    if (bytes == 0) bytes = 256;                       // a zero-element tensor still owns a distinct, aligned buffer
    hipError_t e = hipMalloc(out, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        *out = nullptr;
        return fail(e == hipErrorOutOfMemory ? INCIN_ROCM_ENOMEM : INCIN_ROCM_ERUNTIME,
                    "ROCm allocation of %zu bytes on device %d failed: %s", bytes, dev, hipGetErrorString(e));
    }
    return 0;
}

int incin_rocm_free(int32_t dev, void* ptr)
{
    if (!ptr) return 0;
    if (int rc = use_device(dev)) return rc;
    HIP_TRY(hipFree(ptr), "hipFree");
    return 0;
}

int incin_rocm_memset(int32_t dev, void* dst, int value, size_t bytes)
{
    if (bytes == 0) return 0;
    if (!dst) return fail(INCIN_ROCM_EINVAL, "memset: null pointer");
    if (int rc = use_device(dev)) return rc;
    HIP_TRY(hipMemset(dst, value, bytes), "hipMemset");
    return 0;
}

static int copy(int32_t dev, void* dst, const void* src, size_t bytes, hipMemcpyKind kind, const char* what)
{
    if (bytes == 0) return 0;
    if (!dst || !src) return fail(INCIN_ROCM_EINVAL, "%s: null pointer", what);
    if (int rc = use_device(dev)) return rc;
    HIP_TRY(hipMemcpy(dst, src, bytes, kind), what);
    return 0;
}

int incin_rocm_memcpy_h2d(int32_t dev, void* dst, const void* src, size_t bytes)
{
    return copy(dev, dst, src, bytes, hipMemcpyHostToDevice, "hipMemcpy(host to device)");
}
int incin_rocm_memcpy_d2h(int32_t dev, void* dst, const void* src, size_t bytes)
{
    return copy(dev, dst, src, bytes, hipMemcpyDeviceToHost, "hipMemcpy(device to host)");
}
int incin_rocm_memcpy_d2d(int32_t dev, void* dst, const void* src, size_t bytes)
{
    if (bytes == 0) return 0;
    if (!dst || !src) return fail(INCIN_ROCM_EINVAL, "memcpy_d2d: null pointer");
    if (aligned16(dst) && aligned16(src) && bytes % 16 == 0) {
        // a plain copy kernel on the default stream, then wait: synchronous like the other copies
        if (int rc = use_device(dev)) return rc;
        HIP_TRY(incin_rocm::launch_copy16(dst, src, bytes, nullptr), "copy kernel launch");
        HIP_TRY(hipStreamSynchronize(nullptr), "hipStreamSynchronize");
        return 0;
    }
    return copy(dev, dst, src, bytes, hipMemcpyDeviceToDevice, "hipMemcpy(device to device)");
}

int incin_rocm_copy_strided(int32_t dev, void* dst, const void* src, int32_t rank, const int64_t* shape, const int64_t* strides,
                            int32_t elem_bytes, void* stream)
{
    if (rank < 0 || rank > 8) return fail(INCIN_ROCM_ESHAPE, "copy_strided: rank %d is outside 0..8", rank);
    if (elem_bytes != 2 && elem_bytes != 4) return fail(INCIN_ROCM_EDTYPE, "copy_strided: elements of %d bytes (2 or 4 only)", elem_bytes);
    if (rank > 0 && (!shape || !strides)) return fail(INCIN_ROCM_EINVAL, "copy_strided: null shape or strides");
    incin_rocm::StridedCopyParams p;
    int64_t n = 1;
    for (int a = 0; a < 8; ++a) { p.shape[a] = 1; p.stride[a] = 0; }
    for (int a = 0; a < rank; ++a) {
        if (shape[a] < 0) return fail(INCIN_ROCM_ESHAPE, "copy_strided: negative extent");
        if (shape[a] > 0x7fffffffLL || (n *= shape[a]) > (1LL << 40)) return fail(INCIN_ROCM_ESHAPE, "copy_strided: view too large");
        p.shape[8 - rank + a] = shape[a];
        p.stride[8 - rank + a] = strides[a];
    }
    if (n == 0) return 0;
    if (!dst || !src) return fail(INCIN_ROCM_EINVAL, "copy_strided: null pointer");
    if (((uintptr_t)dst | (uintptr_t)src) % (uintptr_t)elem_bytes) return fail(INCIN_ROCM_EINVAL, "copy_strided: misaligned pointer");
    p.src = (const char*)src;
    p.dst = (char*)dst;
    p.elem = elem_bytes;
    p.outer = 1;
    for (int a = 0; a < 6; ++a) p.outer *= p.shape[a];
    if (int rc = use_device(dev)) return rc;
    HIP_TRY(incin_rocm::launch_copy_strided(p, (hipStream_t)stream), "strided copy launch");
    return 0;
}

int incin_rocm_sum_to_shape(int32_t dev, int32_t dtype, void* dst, const void* src, int32_t rank, const int64_t* src_shape,
                            const int64_t* dst_shape, void* stream)
{
    if (rank < 0 || rank > 8) return fail(INCIN_ROCM_ESHAPE, "sum_to_shape: rank %d is outside 0..8", rank);
    if (dtype != INCIN_ROCM_F32 && dtype != INCIN_ROCM_F16 && dtype != INCIN_ROCM_BF16)
        return fail(INCIN_ROCM_EDTYPE, "sum_to_shape: unsupported dtype tag %d on backend Rocm (f32, f16, bf16 only)", dtype);
    if (rank > 0 && (!src_shape || !dst_shape)) return fail(INCIN_ROCM_EINVAL, "sum_to_shape: null shape");
    incin_rocm::SumToShapeParams p;
    int64_t n_src = 1, n_dst = 1;
    for (int a = 0; a < 8; ++a) { p.src_shape[a] = 1; p.dst_shape[a] = 1; }
    for (int a = 0; a < rank; ++a) {
        if (src_shape[a] < 0 || dst_shape[a] < 0) return fail(INCIN_ROCM_ESHAPE, "sum_to_shape: negative extent");
        if (dst_shape[a] != src_shape[a] && dst_shape[a] != 1)
            return fail(INCIN_ROCM_ESHAPE, "sum_to_shape: axis %d has extent %lld in the source and %lld in the target (the same, or 1)", a,
                        (long long)src_shape[a], (long long)dst_shape[a]);
        if (src_shape[a] > 0x7fffffffLL || (n_src *= src_shape[a]) > (1LL << 40)) return fail(INCIN_ROCM_ESHAPE, "sum_to_shape: source too large");
        n_dst *= dst_shape[a];
        p.src_shape[8 - rank + a] = src_shape[a];
        p.dst_shape[8 - rank + a] = dst_shape[a];
    }
    if (n_dst == 0) return 0;
    if (!dst) return fail(INCIN_ROCM_EINVAL, "sum_to_shape: null pointer");
    if (int rc = use_device(dev)) return rc;
    if (n_dst > 0x7fffffffLL) return fail(INCIN_ROCM_ESHAPE, "sum_to_shape: target too large");
    if (n_src == 0) {       // an empty sum is 0 (the reference starts every sum from the default value)
        HIP_TRY(incin_rocm::launch_zero_rows(dst, dtype == INCIN_ROCM_F32 ? 4 : 2, 1, 1, 1, (int)n_dst, 0, 0, 0, (hipStream_t)stream), "zero fill launch");
        return 0;
    }
    if (!src) return fail(INCIN_ROCM_EINVAL, "sum_to_shape: null pointer");
    p.src = (const char*)src;
    p.dst = (char*)dst;
    p.dtype = dtype;
    HIP_TRY(incin_rocm::launch_sum_to_shape(p, (hipStream_t)stream), "sum_to_shape launch");
    return 0;
}

int incin_rocm_mask_row_limits(int32_t dev, int32_t dtype, const void* mask, const int64_t* shape, const int64_t* strides, int32_t* lims, void* stream)
{
    if (dtype != INCIN_ROCM_F32 && dtype != INCIN_ROCM_F16 && dtype != INCIN_ROCM_BF16)
        return fail(INCIN_ROCM_EDTYPE, "mask_row_limits: unsupported dtype tag %d on backend Rocm (f32, f16, bf16 only)", dtype);
    if (!shape || !strides) return fail(INCIN_ROCM_EINVAL, "mask_row_limits: null shape");
    int64_t rows = 1;
    for (int a = 0; a < 4; ++a) {
        if (shape[a] < 0 || shape[a] > 0x7fffffffLL) return fail(INCIN_ROCM_ESHAPE, "mask_row_limits: extent %lld of axis %d", (long long)shape[a], a);
        if (a < 3) rows *= shape[a];
        if (rows > (1LL << 40)) return fail(INCIN_ROCM_ESHAPE, "mask_row_limits: mask too large");
    }
    if (rows == 0) return 0;
    if (!lims || (!mask && shape[3] > 0)) return fail(INCIN_ROCM_EINVAL, "mask_row_limits: null pointer");
    if (int rc = use_device(dev)) return rc;
    HIP_TRY(incin_rocm::launch_mask_row_limits(mask, dtype, shape, strides, lims, (hipStream_t)stream), "mask_row_limits launch");
    return 0;
}

int incin_rocm_sync(int32_t dev)
{
    if (int rc = use_device(dev)) return rc;
    HIP_TRY(hipDeviceSynchronize(), "hipDeviceSynchronize");
    return 0;
}

int incin_rocm_stream_create(int32_t dev, void** out)
{
    if (!out) return fail(INCIN_ROCM_EINVAL, "stream_create: null output");
    *out = nullptr;
    if (int rc = use_device(dev)) return rc;
    hipStream_t s;
    HIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreateWithFlags");   // default priority
    *out = (void*)s;
    return 0;
}

int incin_rocm_stream_destroy(int32_t dev, void* stream)
{
    if (!stream) return 0;
    if (int rc = use_device(dev)) return rc;
    HIP_TRY(hipStreamDestroy((hipStream_t)stream), "hipStreamDestroy");
    return 0;
}

int incin_rocm_stream_sync(int32_t dev, void* stream)
{
    if (int rc = use_device(dev)) return rc;
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
    return 0;
}

int incin_rocm_event_query(int32_t dev, void* event, int32_t* done)
{
    if (!event || !done) return fail(INCIN_ROCM_EINVAL, "event_query: null argument");
    if (int rc = use_device(dev)) return rc;
    const hipError_t e = hipEventQuery((hipEvent_t)event);
    if (e != hipSuccess && e != hipErrorNotReady) return fail(INCIN_ROCM_ERUNTIME, "ROCm hipEventQuery failed: %s", hipGetErrorString(e));
    *done = e == hipSuccess ? 1 : 0;
    return 0;
}

int incin_rocm_graph_begin(int32_t dev, void* stream)
{
    if (!stream) return fail(INCIN_ROCM_EINVAL, "graph_begin: recording needs a stream of its own, not the default stream");
    if (int rc = use_device(dev)) return rc;
    // thread-local mode: other threads may go on allocating and launching while this one records
    HIP_TRY(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
    return 0;
}

int incin_rocm_graph_end(int32_t dev, void* stream, void** graph_out)
{
    if (!graph_out) return fail(INCIN_ROCM_EINVAL, "graph_end: null output");
    *graph_out = nullptr;
    if (int rc = use_device(dev)) return rc;
    hipGraph_t g = nullptr;
    HIP_TRY(hipStreamEndCapture((hipStream_t)stream, &g), "hipStreamEndCapture");
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess) return fail(INCIN_ROCM_ERUNTIME, "ROCm hipGraphInstantiate failed: %s", hipGetErrorString(e));
    *graph_out = (void*)exec;
    return 0;
}

int incin_rocm_graph_launch(int32_t dev, void* graph, void* stream)
{
    if (!graph) return fail(INCIN_ROCM_EINVAL, "graph_launch: null graph");
    if (int rc = use_device(dev)) return rc;
    HIP_TRY(hipGraphLaunch((hipGraphExec_t)graph, (hipStream_t)stream), "hipGraphLaunch");
    return 0;
}

int incin_rocm_graph_destroy(int32_t dev, void* graph)
{
    if (!graph) return 0;
    if (int rc = use_device(dev)) return rc;
    HIP_TRY(hipGraphExecDestroy((hipGraphExec_t)graph), "hipGraphExecDestroy");
    return 0;
}

int incin_rocm_event_create(int32_t dev, void** out)
{
    if (!out) return fail(INCIN_ROCM_EINVAL, "event_create: null output");
    *out = nullptr;
    if (int rc = use_device(dev)) return rc;
    hipEvent_t e;
    HIP_TRY(hipEventCreate(&e), "hipEventCreate");
    *out = (void*)e;
    return 0;
}

int incin_rocm_event_destroy(int32_t dev, void* event)
{
    if (!event) return 0;
    if (int rc = use_device(dev)) return rc;
    HIP_TRY(hipEventDestroy((hipEvent_t)event), "hipEventDestroy");
    return 0;
}

int incin_rocm_event_record(int32_t dev, void* event, void* stream)
{
    if (!event) return fail(INCIN_ROCM_EINVAL, "event_record: null event");
    if (int rc = use_device(dev)) return rc;
    HIP_TRY(hipEventRecord((hipEvent_t)event, (hipStream_t)stream), "hipEventRecord");
    return 0;
}

int incin_rocm_event_sync(int32_t dev, void* event)
{
    if (!event) return fail(INCIN_ROCM_EINVAL, "event_sync: null event");
    if (int rc = use_device(dev)) return rc;
    HIP_TRY(hipEventSynchronize((hipEvent_t)event), "hipEventSynchronize");
    return 0;
}

int incin_rocm_event_elapsed_ms(int32_t dev, void* start, void* stop, float* out_ms)
{
    if (!start || !stop || !out_ms) return fail(INCIN_ROCM_EINVAL, "event_elapsed_ms: null argument");
    if (int rc = use_device(dev)) return rc;
    HIP_TRY(hipEventElapsedTime(out_ms, (hipEvent_t)start, (hipEvent_t)stop), "hipEventElapsedTime");
    return 0;
}

int incin_rocm_sdpa_workspace(const incin_rocm_sdpa_desc_t* desc, size_t* bytes, int32_t* splits, int32_t* impl_out)
{
    Plan plan;
    if (int rc = make_plan(desc, &plan)) return rc;
    if (bytes) *bytes = plan.ws_bytes;
    if (splits) *splits = plan.splits;
    if (impl_out) *impl_out = plan.impl;
    return 0;
}

// Launches a validated request; the scratch memory is what desc->workspace names.
static int launch_fwd(const incin_rocm_sdpa_desc_t* desc, const Plan& plan, void* stream)
{
    if (plan.ws_bytes > 0) {
        if (!desc->workspace || desc->workspace_bytes < plan.ws_bytes)
            return fail(INCIN_ROCM_EWORKSPACE,
                        "scaled_dot_product_attention: %s needs %zu workspace bytes, %zu given",
                        plan.impl != INCIN_ROCM_IMPL_MFMA ? "split-KV" : desc->add_mask ? "a dense mask on the MFMA kernels" : "the MFMA prefill kernel with the keys split",
                        plan.ws_bytes,
                        desc->workspace ? desc->workspace_bytes : (size_t)0);
        if (!aligned16(desc->workspace)) return fail(INCIN_ROCM_EWORKSPACE, "scaled_dot_product_attention: workspace must be 16-byte aligned");
    }
    if (int rc = use_device(desc->device)) return rc;
    SdpaParams p;
    fill_params(desc, plan, &p);
    hipStream_t s = (hipStream_t)stream;
    hipError_t e;
    switch (plan.impl) {
        case INCIN_ROCM_IMPL_MFMA:
            if (p.mask) {           // block flags of the mask first (and its row limits), on the same stream
                e = incin_rocm::launch_mask_classify(p, desc->dtype, s);
                if (e != hipSuccess) break;
                if (plan.lims_splitkv) {
                    SdpaParams pl = p;
                    pl.num_splits = 1;
                    pl.split_len = (int)((desc->Skv + 255) / 256 * 256);
                    e = incin_rocm::launch_sdpa_decode_f32_limits(pl, s);
                    if (e != hipSuccess) break;
                }
            }
            e = p.Dp == 256                    ? incin_rocm::launch_sdpa_prefill_wide(p, desc->dtype, s)
                : desc->dtype == INCIN_ROCM_F32 ? incin_rocm::launch_sdpa_prefill_f32(p, s)
                                                : incin_rocm::launch_sdpa_prefill_mfma(p, desc->dtype, s);
            break;
        case INCIN_ROCM_IMPL_SPLITKV: e = incin_rocm::launch_sdpa_decode(p, desc->dtype, s); break;
        case INCIN_ROCM_IMPL_SPLITKV_MFMA: e = incin_rocm::launch_sdpa_decode_mfma(p, desc->dtype, s); break;
        default: e = incin_rocm::launch_sdpa_generic(p, desc->dtype, s); break;
    }
    if (e != hipSuccess) return hip_fail(e, "attention kernel launch");
    return 0;
}

int incin_rocm_sdpa_fwd(const incin_rocm_sdpa_desc_t* desc, void* stream)
{
    Plan plan;
    if (int rc = make_plan(desc, &plan)) return rc;
    if (plan.empty) return 0;
    return launch_fwd(desc, plan, stream);
}

// ---- the entry point that allocates nothing ------------------------------------------------------------------
// Scratch memory of incin_rocm_sdpa_fwd_static: part of the code object, so every device the library runs on holds
// its own copy from the moment the code object is loaded there until the process ends.  In host code the array's
// name is only a handle for hipGetSymbolAddress, never a device address: static_scratch_of() asks once per device,
// with that device current, and everything on the host side uses the pointer it returns.
static __device__ __align__(256) unsigned char g_static_scratch[INCIN_ROCM_STATIC_SCRATCH_BYTES];

static int static_scratch_of(int32_t dev, void** out)
{
    static std::mutex mu;
    static void* ptrs[64];
    if (dev < 0 || dev >= 64) return fail(INCIN_ROCM_EDEVICE, "sdpa_fwd_static: device ordinal %d is outside the table of 64", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void* ptr = nullptr;                               // (the caller has made `dev` the current device)
        hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_static_scratch));
        if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(static scratch)");
        if (!ptr) return fail(INCIN_ROCM_ERUNTIME, "ROCm hipGetSymbolAddress(static scratch) returned no address on device %d", dev);
        ptrs[dev] = ptr;
    }
    *out = ptrs[dev];
    return 0;
}

int incin_rocm_sdpa_fwd_static(const incin_rocm_sdpa_desc_t* desc, void* stream)
{
    Plan plan;
    if (int rc = make_plan(desc, &plan)) return rc;
    if (plan.empty) return 0;
    if (plan.ws_bytes > (size_t)INCIN_ROCM_STATIC_SCRATCH_BYTES && plan.impl == INCIN_ROCM_IMPL_MFMA && !desc->add_mask &&
        desc->num_splits == 0) {
        // a prefill launch whose keys the library chose to split, with more partial results than the buffer holds: the
        // same launch without splits needs no scratch memory at all
        incin_rocm_sdpa_desc_t whole = *desc;
        whole.num_splits = 1;
        if (int rc = make_plan(&whole, &plan)) return rc;
    }
    if (plan.ws_bytes > (size_t)INCIN_ROCM_STATIC_SCRATCH_BYTES)
        return fail(INCIN_ROCM_EWORKSPACE,
                    "sdpa_fwd_static: this request needs %zu bytes of scratch memory, the static buffer holds %zu "
                    "(fewer splits, or incin_rocm_sdpa_fwd with a workspace of the caller's)",
                    plan.ws_bytes, (size_t)INCIN_ROCM_STATIC_SCRATCH_BYTES);
    incin_rocm_sdpa_desc_t d = *desc;
    d.workspace = nullptr;
    d.workspace_bytes = 0;
    if (plan.ws_bytes > 0) {
        if (int rc = use_device(desc->device)) return rc;
        void* scratch = nullptr;
        if (int rc = static_scratch_of(desc->device, &scratch)) return rc;
        d.workspace = scratch;
        d.workspace_bytes = (size_t)INCIN_ROCM_STATIC_SCRATCH_BYTES;
    }
    return launch_fwd(&d, plan, stream);
}


int incin_rocm_matrix_rate(int32_t dev, const void* operands, void* sink, int32_t mix, int32_t iterations, double* flops, void* stream)
{
    if (!operands || !sink || !flops) return fail(INCIN_ROCM_EINVAL, "matrix_rate: null pointer");
    if (mix < 0 || mix > 1 || iterations < 1 || iterations > (1 << 24)) return fail(INCIN_ROCM_EINVAL, "matrix_rate: mix is 0 or 1, iterations 1 .. 2^24");
    if (int rc = use_device(dev)) return rc;
    const hipError_t e = incin_rocm::launch_matrix_rate(operands, sink, mix, iterations, flops, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "matrix rate launch");
    return 0;
}

int incin_rocm_read_rate(int32_t dev, const void* src, size_t bytes, int32_t nontemporal, void* sink, void* stream)
{
    if (!src || !sink) return fail(INCIN_ROCM_EINVAL, "read_rate: null pointer");
    if (bytes == 0 || bytes % ((size_t)4096 * 32768) != 0) return fail(INCIN_ROCM_EINVAL, "read_rate: bytes is a positive multiple of 128 MiB");
    if (!aligned16(src)) return fail(INCIN_ROCM_EINVAL, "read_rate: src must be 16-byte aligned");
    if (int rc = use_device(dev)) return rc;
    const hipError_t e = incin_rocm::launch_read_rate(src, sink, bytes, nontemporal != 0, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "read rate launch");
    return 0;
}

int incin_rocm_lds_fill(int32_t dev, uint32_t pattern, void* sink, void* stream)
{
    if (!sink) return fail(INCIN_ROCM_EINVAL, "lds_fill: null pointer");
    if (int rc = use_device(dev)) return rc;
    const hipError_t e = incin_rocm::launch_lds_fill(sink, pattern, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "lds fill launch");
    return 0;
}

size_t incin_rocm_sizeof_sdpa_bwd_desc(void) { return sizeof(incin_rocm_sdpa_bwd_desc_t); }

// Validates a backward request; *empty is set when there is nothing to compute, *kind says which kernels take it:
// 0 the generic ones, 1 the 16-bit matrix-core ones, 2 the IEEE-f32 matrix-core ones.
static int check_bwd(const incin_rocm_sdpa_bwd_desc_t* bd, bool* empty, int* kind)
{
    static const char* OP = "scaled_dot_product_attention backward";
    if (!bd) return fail(INCIN_ROCM_EINVAL, "%s: null descriptor", OP);
    const incin_rocm_sdpa_desc_t* d = &bd->fwd;
    Plan plan;
    {
        incin_rocm_sdpa_desc_t any = *d;            // shapes, dtype, strides, mask: whatever some forward kernel accepts
        any.impl = INCIN_ROCM_IMPL_AUTO;
        if (int rc = make_plan(&any, &plan)) return rc;
    }
    *empty = plan.empty || d->Skv == 0;
    *kind = 0;
    if (*empty) return 0;
    if (!d->lse) return fail(INCIN_ROCM_EINVAL, "%s: fwd.lse (the forward's row normalisers) is required", OP);
    if (!bd->d_o || !bd->d_q || !bd->d_k || !bd->d_v) return fail(INCIN_ROCM_EINVAL, "%s: null gradient pointer", OP);
    if (d->D > 256 || d->Dv > 256) return fail(INCIN_ROCM_EUNSUPPORTED, "%s: D and Dv up to 256", OP);

    // both matrix-core families: whole rows move as 16-byte vectors, tiles are addressed with 32-bit byte offsets
    const bool f32 = d->dtype == INCIN_ROCM_F32;
    const int vec = f32 ? 4 : 8;
    // (head dimensions up to 128 in whole 16-byte vectors, D and Dv not necessarily equal: zero-padded into the 64 / 128 instances)
    bool ok = d->D > 0 && d->D <= 128 && d->Dv <= 128 && d->D % vec == 0 && d->Dv % vec == 0 && std::isfinite(d->scale) && (f32 || d->scale > 0.0f);
    ok = ok && fast_layout_ok(d, vec) && aligned16(bd->d_o) && aligned16(bd->d_q) && aligned16(bd->d_k) && aligned16(bd->d_v);
    for (int a = 0; a < 3; ++a)
        ok = ok && bd->d_o_stride[a] % vec == 0 && bd->d_q_stride[a] % vec == 0 && bd->d_k_stride[a] % vec == 0 && bd->d_v_stride[a] % vec == 0;
    const int64_t big = f32 ? (1 << 22) : (1 << 24);
    ok = ok && d->q_stride[2] >= 0 && d->q_stride[2] < big && d->k_stride[2] >= 0 && d->k_stride[2] < big && d->v_stride[2] >= 0 &&
         d->v_stride[2] < big && bd->d_o_stride[2] >= 0 && bd->d_o_stride[2] < big;
    if (d->add_mask)      // a tile's mask values are addressed with 32-bit byte offsets from the tile's first row
        ok = ok && d->mask_stride[2] >= 0 && d->mask_stride[3] >= 0 &&
             (64 * d->mask_stride[2] + (d->Skv > 0 ? d->Skv - 1 : 0) * d->mask_stride[3] + 1) * (f32 ? 4 : 2) < (int64_t)0x7fffffff;
    const int fast = f32 ? 2 : 1;
    if (d->impl == INCIN_ROCM_IMPL_AUTO) *kind = ok ? fast : 0;
    else if (d->impl == INCIN_ROCM_IMPL_GENERIC) *kind = 0;
    else if (d->impl == INCIN_ROCM_IMPL_MFMA) {
        if (!ok)
            return fail(INCIN_ROCM_EUNSUPPORTED, "%s: the MFMA kernels need D and Dv <= 128 in whole 16-byte vectors, a finite scale (f16 / bf16: "
                        "positive), 64 rows of a dense mask within 2 GiB, and rows 16-byte aligned with strides that are multiples of 16 bytes below 2^%d elements",
                        OP, f32 ? 22 : 24);
        *kind = fast;
    } else
        return fail(INCIN_ROCM_EUNSUPPORTED, "%s: impl is one of AUTO, GENERIC, MFMA", OP);
    return 0;
}

// Workspace of a backward call: two f32 per query row; with a dense mask on the matrix-core kernels also the mask's
// block flags (one byte per 32 rows x 32 keys, as the forward's: hidden blocks are skipped), behind them.
static size_t bwd_rows_bytes(const incin_rocm_sdpa_desc_t* d) { return (2 * (size_t)(d->B * d->Hq * d->Sq) * sizeof(float) + 255) / 256 * 256; }
static size_t bwd_flags_bytes(const incin_rocm_sdpa_desc_t* d, int kind)
{
    if (kind == 0 || !d->add_mask) return 0;
    const int64_t nbh = (d->mask_stride[0] ? d->B : 1) * (d->mask_stride[1] ? d->Hq : 1);
    return (size_t)(nbh * ((d->Sq + 31) / 32) * ((d->Skv + 31) / 32) + 255) / 256 * 256;
}

// Matrix-core kernels: into how many workgroups the key tiles of a block of 128 rows (dQ kernel, which = 0) or the query
// tiles of a block of 128 keys (dK/dV kernel, which = 1) are dealt.  A launch of half a round of workgroups or less leaves
// most of the device idle - under a causal mask every SIMD has one wavefront and all wait for the one with the longest
// walk - so its tiles go to 2 workgroups (up to half a round) or 4 (up to a quarter), each with at least four tiles of 64 to
// walk; the sums meet in planes of the workspace and a pass adds them (sdpa_bwd.h).
// f32 (kind 2), both kernels.  Measured, whole call, against one workgroup per block (causal, with the dQ kernel on its side
// stream either way): 8 heads x 1024 keys 0.36 (D = 64, 4 parts) / 0.56 (128); 32 heads x 1024 0.86 (D = 64, 2 parts: config
// 2's shape) and 0.99 at D = 128 (a full round: not split); 16 query heads on 4 KV heads x 2048 0.38 / 0.41; from a full round
// on 1.0 - 1.13: not split.
// 16-bit storage (kind 1), the dK/dV kernel only - a workgroup of it fills a compute unit, a round is one per compute unit,
// and with grouped queries a key block walks every head of its group: few KV heads on a device (a model's KV heads
// divided over devices) leave most compute units without a block.  Measured, whole call, bf16 causal D = 128: 8 query heads on
// 1 KV head x 8192 keys 1.66 -> 0.73 ms (4 parts; 2: 0.54 of the time, 8: 0.46), x 4096 0.84 -> 0.25 (8 parts: 0.28); 16 on 2
// x 8192 0.72 (2 parts; 4: 0.85); 32 on 4 x 4096 0.80 (2); D = 64 8 on 1 x 8192 0.40; not worth it for short walks (8 heads x
// 2048 keys without groups, 32 tiles per block: 1.19 in 2 parts) - a part keeps at least 64 tiles.  The kernel takes up to 8
// parts, the rule stops at 4.
static int bwd_parts(const incin_rocm_sdpa_desc_t* d, int kind, int which)
{
    if (kind == 0 || (kind == 1 && which == 0)) return 1;
    const char* forced = getenv("INCIN_ROCM_BWD_PARTS");      // (1, 2, 4 or 8 for every kernel that takes parts: a test knob)
    const int64_t blocks = which == 0 ? ((d->Sq + 127) / 128) * d->Hq * d->B : ((d->Skv + 127) / 128) * d->Hkv * d->B;
    const int64_t slots = (int64_t)(kind == 1 || d->D > 64 || d->Dv > 64 ? 1 : 2) * compute_units_of(d->device);
    const int64_t walk = (which == 0 ? d->Skv : d->Sq * (d->Hq / d->Hkv)) / 64;
    int parts = 1;
    const int f = forced ? atoi(forced) : 0;
    if (f == 1 || f == 2 || f == 4 || f == 8) {
        parts = std::min(f, kind == 1 ? 8 : 4);
        while (parts > 1 && walk < 4 * parts) parts >>= 1;
        return parts;
    }
    while (parts < 4 && 2 * parts * blocks <= slots) parts *= 2;
    // (f32: four tiles per part are enough to pay for the planes; 16-bit storage, whose tiles take an eighth of the time: 64)
    while (parts > 1 && walk < (kind == 1 ? 64 : 4) * parts) parts >>= 1;
    // 16-bit storage, up to a full round of key blocks with very long walks (8 query heads on 1 KV head x 32768 keys: 256 blocks
    // of up to 4096 tiles): under a causal mask the longest walk is twice the average and the round ends with it - four parts
    // make four rounds of shorter items (10.2 -> 7.3 ms there; 16 heads on 2 x 16384, 2048 tiles: 0.84; at 512 tiles 1.05)
    if (kind == 1 && parts == 1 && blocks <= slots && walk >= 2048 && (d->causal || d->add_mask)) parts = 4;
    // ... and two parts already from 256 tiles on when the dQ kernel is not running beside this one to fill the compute units the
    // short walks leave idle (the launcher's rule: D = 64, or at most four dQ blocks per compute unit).  One sequence of 4096
    // tokens, D = 128: 64 query heads on 8 KV heads 1.28 -> 1.01 ms, 128 on 8 2.62 -> 1.91, 48 on 8 0.97 -> 0.79, 2 x 32 on 4 1.29 ->
    // 1.02; with the dQ kernel beside it (2 x 8 on 2 x 8192) two parts cost 19 %.
    const bool dq_beside = (d->D <= 64 && d->Dv <= 64) || ((d->Sq + 127) / 128) * d->Hq * d->B <= 4 * (int64_t)compute_units_of(d->device);
    if (kind == 1 && parts == 1 && blocks <= slots && walk >= 256 && !dq_beside && (d->causal || d->add_mask)) parts = 2;
    return parts;
}
static size_t round256(size_t n) { return (n + 255) / 256 * 256; }
static size_t bwd_planes_bytes(const incin_rocm_sdpa_desc_t* d, int kind, int parts_q, int parts_kv)
{
    const size_t q = round256((size_t)(d->B * d->Hq * d->Sq * d->D) * sizeof(float));
    const size_t k = round256((size_t)(d->B * d->Hkv * d->Skv * d->D) * sizeof(float));
    const size_t v = round256((size_t)(d->B * d->Hkv * d->Skv * d->Dv) * sizeof(float));
    // (f32: part 0 writes the gradient itself; 16-bit storage: every part of a divided walk writes a plane)
    const int planes_kv = kind == 1 ? (parts_kv > 1 ? parts_kv : 0) : parts_kv - 1;
    return (size_t)(parts_q - 1) * q + (size_t)planes_kv * (k + v);
}

int incin_rocm_sdpa_bwd_workspace(const incin_rocm_sdpa_bwd_desc_t* bd, size_t* bytes)
{
    if (!bytes) return fail(INCIN_ROCM_EINVAL, "scaled_dot_product_attention backward: null output");
    *bytes = 0;
    bool empty = false;
    int kind = 0;
    if (int rc = check_bwd(bd, &empty, &kind)) return rc;
    if (!empty) {
        const size_t flags = bwd_flags_bytes(&bd->fwd, kind);
        const size_t planes = bwd_planes_bytes(&bd->fwd, kind, bwd_parts(&bd->fwd, kind, 0), bwd_parts(&bd->fwd, kind, 1));
        *bytes = flags || planes ? bwd_rows_bytes(&bd->fwd) + flags + planes : 2 * (size_t)(bd->fwd.B * bd->fwd.Hq * bd->fwd.Sq) * sizeof(float);
    }
    return 0;
}

int incin_rocm_sdpa_bwd(const incin_rocm_sdpa_bwd_desc_t* bd, void* stream)
{
    bool empty = false;
    int kind = 0;
    if (int rc = check_bwd(bd, &empty, &kind)) return rc;
    if (empty) {
        // No element to write - except with queries but no keys: the output is zeros whatever q holds, so d_q is zero
        // (the reference's tape gives zeros there), and it is promised to be fully overwritten.
        const incin_rocm_sdpa_desc_t* d = &bd->fwd;
        if (d->Skv == 0 && d->B > 0 && d->Hq > 0 && d->Sq > 0 && d->D > 0) {
            if (!bd->d_q) return fail(INCIN_ROCM_EINVAL, "scaled_dot_product_attention backward: null gradient pointer");
            if (int rc = use_device(d->device)) return rc;
            HIP_TRY(incin_rocm::launch_zero_rows(bd->d_q, (int)dtype_size(d->dtype), (int)d->B, (int)d->Hq, (int)d->Sq, (int)d->D,
                                                 bd->d_q_stride[0], bd->d_q_stride[1], bd->d_q_stride[2], (hipStream_t)stream),
                    "gradient clear launch");
        }
        return 0;
    }
    const size_t flag_bytes = bwd_flags_bytes(&bd->fwd, kind);
    const int parts_q = bwd_parts(&bd->fwd, kind, 0), parts_kv = bwd_parts(&bd->fwd, kind, 1);
    const size_t plane_bytes = bwd_planes_bytes(&bd->fwd, kind, parts_q, parts_kv);
    const size_t need = flag_bytes || plane_bytes ? bwd_rows_bytes(&bd->fwd) + flag_bytes + plane_bytes
                                   : 2 * (size_t)(bd->fwd.B * bd->fwd.Hq * bd->fwd.Sq) * sizeof(float);      // two f32 per query row (+ the mask's block flags, + the planes of a split call)
    if (!bd->workspace || bd->workspace_bytes < need || !aligned16(bd->workspace))
        return fail(INCIN_ROCM_EWORKSPACE, "scaled_dot_product_attention backward: %zu workspace bytes needed (16-byte aligned), %zu given",
                    need, bd->workspace ? bd->workspace_bytes : (size_t)0);
    if (int rc = use_device(bd->fwd.device)) return rc;
    Plan plan;
    plan.impl = INCIN_ROCM_IMPL_GENERIC;
    plan.splits = 1;
    plan.split_len = (int)bd->fwd.Skv;
    incin_rocm::SdpaBwdParams bp;
    memset(&bp, 0, sizeof(bp));
    fill_params(&bd->fwd, plan, &bp.f);
    bp.d_o = bd->d_o; bp.d_q = bd->d_q; bp.d_k = bd->d_k; bp.d_v = bd->d_v;
    bp.neg_l2 = (float*)bd->workspace;
    bp.neg_delta = bp.neg_l2 + bd->fwd.B * bd->fwd.Hq * bd->fwd.Sq;
    bp.do_sb = bd->d_o_stride[0]; bp.do_sh = bd->d_o_stride[1]; bp.do_ss = bd->d_o_stride[2];
    bp.dq_sb = bd->d_q_stride[0]; bp.dq_sh = bd->d_q_stride[1]; bp.dq_ss = bd->d_q_stride[2];
    bp.dk_sb = bd->d_k_stride[0]; bp.dk_sh = bd->d_k_stride[1]; bp.dk_ss = bd->d_k_stride[2];
    bp.dv_sb = bd->d_v_stride[0]; bp.dv_sh = bd->d_v_stride[1]; bp.dv_ss = bd->d_v_stride[2];
    bp.f.mask_flags = nullptr;
    bp.f.mask_lims = nullptr;
    bp.parts_q = parts_q;
    bp.parts_kv = parts_kv;
    if (plane_bytes) {
        const incin_rocm_sdpa_desc_t* d = &bd->fwd;
        char* at = (char*)bd->workspace + bwd_rows_bytes(d) + flag_bytes;
        bp.part_dq = (float*)at;
        at += (size_t)(parts_q - 1) * round256((size_t)(d->B * d->Hq * d->Sq * d->D) * sizeof(float));
        bp.part_dk = (float*)at;
        at += (size_t)(kind == 1 ? parts_kv : parts_kv - 1) * round256((size_t)(d->B * d->Hkv * d->Skv * d->D) * sizeof(float));
        bp.part_dv = (float*)at;
    }
    if (flag_bytes) {
        if (((bd->fwd.Sq + 31) / 32) > 65535 || (bd->fwd.mask_stride[0] ? bd->fwd.B : 1) * (bd->fwd.mask_stride[1] ? bd->fwd.Hq : 1) > 65535)
            return fail(INCIN_ROCM_ESHAPE, "scaled_dot_product_attention backward: mask too large for one launch of the matrix-core kernels");
        bp.f.mask_flags = (const uint8_t*)bd->workspace + bwd_rows_bytes(&bd->fwd);
        hipError_t ec = incin_rocm::launch_mask_classify(bp.f, bd->fwd.dtype, (hipStream_t)stream);
        if (ec != hipSuccess) return hip_fail(ec, "mask classification launch");
    }
    hipError_t e = kind == 2   ? incin_rocm::launch_sdpa_bwd_f32(bp, (hipStream_t)stream)
                   : kind == 1 ? incin_rocm::launch_sdpa_bwd_mfma(bp, bd->fwd.dtype, (hipStream_t)stream)
                               : incin_rocm::launch_sdpa_bwd_generic(bp, bd->fwd.dtype, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "attention backward launch");
    return 0;
}

size_t incin_rocm_sizeof_kv_append_desc(void) { return sizeof(incin_rocm_kv_append_desc_t); }

int incin_rocm_kv_append(const incin_rocm_kv_append_desc_t* d, void* stream)
{
    if (!d) return fail(INCIN_ROCM_EINVAL, "kv_append: null descriptor");
    if (d->dtype != INCIN_ROCM_F32 && d->dtype != INCIN_ROCM_F16 && d->dtype != INCIN_ROCM_BF16)
        return fail(INCIN_ROCM_EDTYPE, "kv_append: dtype %d is not one of f32, f16, bf16", (int)d->dtype);
    if (d->B < 0 || d->Hkv < 0 || d->S_new < 0 || d->S_max < 0 || d->D < 0 || d->Dv < 0)
        return fail(INCIN_ROCM_ESHAPE, "kv_append: negative extent");
    const int64_t lim = 0x7fffffffLL;
    if (d->B > lim || d->Hkv > lim || d->S_new > lim || d->S_max > lim || d->D > (1 << 20) || d->Dv > (1 << 20) ||
        d->B * d->Hkv * d->S_new > lim)
        return fail(INCIN_ROCM_ESHAPE, "kv_append: extent exceeds 2^31-1");
    if (d->B == 0 || d->Hkv == 0 || d->S_new == 0) return 0;
    if (!d->k_new || !d->v_new || !d->k_cache || !d->v_cache || !d->kv_lens)
        return fail(INCIN_ROCM_EINVAL, "kv_append: null operand");
    if (int rc = use_device(d->device)) return rc;
    const int elem = d->dtype == INCIN_ROCM_F32 ? 4 : 2;
    incin_rocm::KvAppendParams p;
    p.k_new = (const char*)d->k_new; p.v_new = (const char*)d->v_new;
    p.k_cache = (char*)d->k_cache; p.v_cache = (char*)d->v_cache;
    p.kv_lens = d->kv_lens;
    p.kn_sb = d->k_new_stride[0]; p.kn_sh = d->k_new_stride[1]; p.kn_ss = d->k_new_stride[2];
    p.vn_sb = d->v_new_stride[0]; p.vn_sh = d->v_new_stride[1]; p.vn_ss = d->v_new_stride[2];
    p.kc_sb = d->k_cache_stride[0]; p.kc_sh = d->k_cache_stride[1]; p.kc_ss = d->k_cache_stride[2];
    p.vc_sb = d->v_cache_stride[0]; p.vc_sh = d->v_cache_stride[1]; p.vc_ss = d->v_cache_stride[2];
    p.B = (int32_t)d->B; p.Hkv = (int32_t)d->Hkv; p.S_new = (int32_t)d->S_new; p.S_max = (int32_t)d->S_max;
    p.k_row_bytes = (int32_t)(d->D * elem); p.v_row_bytes = (int32_t)(d->Dv * elem); p.elem = elem;
    // 16-byte copies need every row start and every row length to be a multiple of 16 bytes
    auto mult16 = [&](int64_t stride_elems) { return (stride_elems * elem) % 16 == 0; };
    bool vec16 = p.k_row_bytes % 16 == 0 && p.v_row_bytes % 16 == 0 && (uintptr_t)d->k_new % 16 == 0 && (uintptr_t)d->v_new % 16 == 0 &&
                 (uintptr_t)d->k_cache % 16 == 0 && (uintptr_t)d->v_cache % 16 == 0;
    for (int i = 0; i < 3; ++i)
        vec16 = vec16 && mult16(d->k_new_stride[i]) && mult16(d->v_new_stride[i]) && mult16(d->k_cache_stride[i]) && mult16(d->v_cache_stride[i]);
    HIP_TRY(incin_rocm::launch_kv_append(p, vec16, (hipStream_t)stream), "kv_append launch");
    return 0;
}

}  // extern "C"
