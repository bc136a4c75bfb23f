// Launch parameters of the copy kernels (copy.hip), shared with the C ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace incin_rocm {

struct StridedCopyParams {
    const char* src;
    char* dst;
    int64_t shape[8];      // right-aligned: shape[7] is the last axis; leading axes of extent 1 pad the front
    int64_t stride[8];     // source strides in elements
    int64_t outer;         // product of shape[0..5]
    int32_t elem;          // bytes per element: 2 or 4
};

// sum_to_shape: source and destination shapes right-aligned to 8 axes, both dense; dst_shape[a] is src_shape[a] or 1
struct SumToShapeParams {
    const char* src;
    char* dst;
    int64_t src_shape[8];
    int64_t dst_shape[8];
    int32_t dtype;         // 0 f32, 1 f16, 2 bf16
};

hipError_t launch_copy16(void* dst, const void* src, size_t bytes, hipStream_t stream);
hipError_t launch_copy_strided(const StridedCopyParams& p, hipStream_t stream);
hipError_t launch_sum_to_shape(const SumToShapeParams& p, hipStream_t stream);
hipError_t launch_zero_rows(void* base, int elem, int B, int H, int S, int row_elems, int64_t sb, int64_t sh, int64_t ss, hipStream_t stream);

}  // namespace incin_rocm
