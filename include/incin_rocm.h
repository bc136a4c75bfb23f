/*
 * incin_rocm.h -- C ABI of the MI355X (gfx950) attention library that backs an
 * opt-in `rocm` backend of incin-backends.
 *
 * Every entry point returns 0 on success or one of the INCIN_ROCM_E* codes; the
 * text of the last failure on the calling thread is returned by
 * incin_rocm_last_error().  No C++ exception, torch type or HIP type crosses
 * this boundary: plain pointers, sizes and fixed-width integers only.
 *
 * What each entry point stands in for in the reference (paths relative to the
 * reference checkout) is cited on its declaration.  The reference's GPU backends
 * reach their driver through the `cudarc` crate; the same call shapes are what a
 * Rust `incin-rocm-sys` crate binds here.
 */
#ifndef INCIN_ROCM_H
#define INCIN_ROCM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define INCIN_ROCM_ABI_VERSION 11

/* ---- status codes (mapped to incin_core::Error variants by the Rust side;
 *      crates/incin-core/src/err.rs:109-223) --------------------------------- */
enum {
    INCIN_ROCM_OK = 0,
    INCIN_ROCM_EINVAL = 1,        /* null pointer / malformed descriptor  -> Error::Msg                    */
    INCIN_ROCM_ESHAPE = 2,        /* shape or stride rule violated        -> Error::ShapeMismatch          */
    INCIN_ROCM_EDTYPE = 3,        /* dtype outside {f32,f16,bf16}         -> Error::UnsupportedDType       */
    INCIN_ROCM_EDEVICE = 4,       /* bad ordinal / no device              -> Error::InvalidDeviceOrdinal   */
    INCIN_ROCM_ENOMEM = 5,        /* device allocation failed             -> Error::OutOfMemory            */
    INCIN_ROCM_EWORKSPACE = 6,    /* workspace missing or too small       -> Error::Msg                    */
    INCIN_ROCM_EUNSUPPORTED = 7,  /* valid request with no kernel         -> Error::UnsupportedBackendOperation */
    INCIN_ROCM_ERUNTIME = 8       /* HIP call failed                      -> Error::Msg("ROCm ... failed")  */
};

/* dtype tags: the float subset of DTypeId (crates/incin-core/src/tensor/dtype.rs:10-101) */
enum { INCIN_ROCM_F32 = 0, INCIN_ROCM_F16 = 1, INCIN_ROCM_BF16 = 2 };

/* kernel selection for incin_rocm_sdpa_desc_t.impl */
enum {
    INCIN_ROCM_IMPL_AUTO = 0,
    INCIN_ROCM_IMPL_GENERIC = 1,   /* fp32-FMA tiled kernel: any dtype, D and Dv <= 256, dense masks     */
    INCIN_ROCM_IMPL_MFMA = 2,      /* MFMA prefill kernels: D and Dv <= 128 in whole 16-byte vectors (instances for 64 and 128; smaller
                                      and unequal head dimensions are zero-padded into LDS); bf16/f16 (scale > 0) and IEEE-f32
                                      matrix instructions for f32; dense mask allowed.  bf16/f16 also above 128, up to 256
                                      (an instance for 256, any finite scale; a dense mask with 8-byte aligned rows)  */
    INCIN_ROCM_IMPL_SPLITKV = 3,   /* vector-ALU split-KV decode kernel + combine: D == Dv in {64,128}, few query rows; dense mask allowed */
    INCIN_ROCM_IMPL_MFMA64 = 4,    /* retired (a prefill kernel with 64 query rows per wavefront): refused with INCIN_ROCM_EUNSUPPORTED */
    INCIN_ROCM_IMPL_SPLITKV_MFMA = 5 /* split-KV kernels on the matrix cores + combine: D and Dv <= 256 in whole 16-byte vectors (instances for
                                      64, 128 and 256), Sq <= 64 - any Sq when a head dimension is above 128, which only these kernels
                                      cover; the rows that share a KV head (query heads of the group x query positions) go through
                                      them 32 or 64 at a time (bf16/f16), 16 or 32 at a time on IEEE-f32 matrix instructions (f32) */
};

/* Thread-local message of the last failing call on this thread ("" if none).
 * Replaces the `Display` text cudarc errors carry into Error::Msg
 * (crates/incin-backends/src/cuda/ops/matmul.rs:89). */
const char* incin_rocm_last_error(void);
int incin_rocm_abi_version(void);
/* sizeof the two structs below as this build sees them, so a binding can check its mirrors. */
size_t incin_rocm_sizeof_sdpa_desc(void);
size_t incin_rocm_sizeof_device_info(void);

/* ---- device table -----------------------------------------------------------
 * Replaces the per-ordinal context cache of the CUDA backend
 * (crates/incin-backends/src/cuda/gpu.rs:99-152: `CudaContext::new(ordinal)`
 * behind a process-wide map) and `detect::probe`
 * (crates/incin-backends/src/detect.rs:69-77). */
typedef struct {
    char name[64];
    char arch[32];              /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
    int32_t compute_units;
    int32_t clock_khz;          /* max engine clock */
    int32_t memory_clock_khz;
    int32_t memory_bus_bits;
    int32_t lds_bytes_per_block;
    int32_t wavefront_size;
    uint64_t hbm_bytes;
} incin_rocm_device_info_t;

int incin_rocm_device_count(int32_t* out);
int incin_rocm_device_info(int32_t dev, incin_rocm_device_info_t* out);

/* ---- buffers ----------------------------------------------------------------
 * Replace CudaBuffer allocation and the H2D / D2H copies behind
 * Backend::from_bytes / Backend::to_bytes
 * (crates/incin-backends/src/cuda/storage.rs:24-59,
 *  crates/incin-backends/src/cuda/backend.rs:1905-1937, 2007-2045).
 * Allocations are at least 256-byte aligned (cuda/storage.rs:18).  Copies are
 * synchronous with respect to the host, as the reference's are. */
int incin_rocm_alloc(int32_t dev, size_t bytes, void** out);
int incin_rocm_free(int32_t dev, void* ptr);
int incin_rocm_memset(int32_t dev, void* dst, int value, size_t bytes);
int incin_rocm_memcpy_h2d(int32_t dev, void* dst, const void* src, size_t bytes);
int incin_rocm_memcpy_d2h(int32_t dev, void* dst, const void* src, size_t bytes);
int incin_rocm_memcpy_d2d(int32_t dev, void* dst, const void* src, size_t bytes);
/* Logical (row-major) contents of a strided view written densely to `dst`: what CpuStorage::contiguous does on the
 * host (crates/incin-backends/src/cpu/storage.rs:407-440), here one kernel enqueued on `stream`.  `shape` and `strides`
 * (elements; 0 on a broadcast axis, negative allowed) have `rank` <= 8 entries, `src` points at the view's first
 * element, elements are 2 or 4 bytes.  The backend uses it for operands of attention whose last axis is strided
 * (a transposed view). */
int incin_rocm_copy_strided(int32_t dev, void* dst, const void* src, int32_t rank, const int64_t* shape, const int64_t* strides,
                            int32_t elem_bytes, void* stream);
/* Gradient of a broadcast operand: `src` (dense, `src_shape`) summed down to `dst` (dense, `dst_shape`), where
 * dst_shape[a] is src_shape[a] or 1 - the axes with 1 are summed away.  Replaces `unbroadcast`
 * (crates/incin-backends/src/cpu/tape.rs:243-265; `sum_dim_keepdim` :283-317): axis after axis from the left, each in
 * ascending order, f32 partial sums (16-bit storage is rounded once at the end).  rank <= 8; a caller with fewer leading
 * axes in the target pads its shape with 1s.  dtype: INCIN_ROCM_F32 / F16 / BF16.  Enqueued on `stream`. */
int incin_rocm_sum_to_shape(int32_t dev, int32_t dtype, void* dst, const void* src, int32_t rank, const int64_t* src_shape,
                            const int64_t* dst_shape, void* stream);
/* What a mask tensor of zeros and -inf states, row by row.  The reference's operator takes its mask as a tensor only
 * (crates/incin-backends/src/cpu/ops/shape_ops.rs:1262-1266) and its callers build the causal mask as
 * full(-inf).triu(1) and key padding as 0 / -inf per key: every row of such a mask is n zeros followed by -inf.  For a mask
 * of shape [A0, A1, rows, Skv] (`shape`, `strides` in elements, 0 on a repeated axis) this writes one int per
 * (a0, a1, row), in that order, to `lims`: n if the row has that form (n = Skv: all zeros, n = 0: all -inf), else -1.
 * A backend that reads the result back can state the mask as `causal` / `kv_lens` in the descriptors (forward and backward)
 * instead of passing the tensor.  Enqueued on `stream`; a row with Skv = 0 gets 0. */
int incin_rocm_mask_row_limits(int32_t dev, int32_t dtype, const void* mask, const int64_t* shape, const int64_t* strides, int32_t* lims,
                               void* stream);
int incin_rocm_sync(int32_t dev);      /* waits for the device's default stream and any stream created here */

/* ---- streams and events -------------------------------------------------------
 * The reference launches on cudarc's per-context default stream
 * (crates/incin-backends/src/cuda/ops/matmul.rs:57-90); a NULL stream here means
 * the same.  Streams are created at default priority only.  Events exist so a
 * caller can time launches on the stream they were issued to. */
int incin_rocm_stream_create(int32_t dev, void** out);
int incin_rocm_stream_destroy(int32_t dev, void* stream);
int incin_rocm_stream_sync(int32_t dev, void* stream);
int incin_rocm_event_create(int32_t dev, void** out);
int incin_rocm_event_destroy(int32_t dev, void* event);
int incin_rocm_event_record(int32_t dev, void* event, void* stream);
int incin_rocm_event_sync(int32_t dev, void* event);
/* *done = 1 once everything recorded before the event has finished, else 0 (never blocks).  What a stream-ordered
 * allocator needs to hand a released buffer to another stream: the reference's CUDA buffers are allocated and freed
 * in stream order by its driver crate (crates/incin-backends/src/cuda/storage.rs:171-177, 225-233). */
int incin_rocm_event_query(int32_t dev, void* event, int32_t* done);
int incin_rocm_event_elapsed_ms(int32_t dev, void* start, void* stop, float* out_ms);

/* ---- launch graphs ------------------------------------------------------------
 * No counterpart in the reference (its backends launch eagerly).  For callers that replay a fixed sequence of
 * launches, a decode loop for one: everything enqueued on `stream` between begin and end is recorded instead of
 * run, and the recording is replayed with incin_rocm_graph_launch.  incin_rocm_sdpa_fwd can be recorded: it
 * neither allocates nor clears memory (the workspace is the caller's).  The allocating and copying entry points
 * above must not be called on a stream that is recording. */
int incin_rocm_graph_begin(int32_t dev, void* stream);
int incin_rocm_graph_end(int32_t dev, void* stream, void** graph_out);
int incin_rocm_graph_launch(int32_t dev, void* graph, void* stream);
int incin_rocm_graph_destroy(int32_t dev, void* graph);

/* ---- attention forward --------------------------------------------------------
 * Replaces CpuBackendImpl::scaled_dot_product_attention
 * (crates/incin-backends/src/cpu/ops/shape_ops.rs:1245-1269), the only
 * implementation of TensorOps::scaled_dot_product_attention
 * (crates/incin-core/src/tensor/backend.rs:485-492):
 *
 *     o = softmax(q k^T * scale + mask) v        row-wise softmax over keys
 *
 * The caller has already collapsed the operator's leading axes into
 * (B, Hkv, G) by the reference's batch-broadcast rule
 * (crates/incin-backends/src/cpu/ops/matmul.rs:198-221): query head hq reads
 * key/value head hq / (Hq / Hkv); a broadcast axis is a stride of 0.
 *
 * Masking.  The reference knows one mask form, an additive tensor broadcast
 * against the scores (shape_ops.rs:1262-1266).  `add_mask` is that tensor.
 * `causal` and `kv_lens` state, without materialising them, the two additive
 * masks of 0 / -inf that callers build most: key j is masked (as if -inf were
 * added) when  causal != 0 and j > i + (Skv - Sq),  or  kv_lens != NULL and
 * j >= kv_lens[b].  All three may be combined.  A query row with every key
 * masked yields NaN, as the reference's softmax does (-inf - -inf).
 *
 * Padded batches.  `q_lens` has no counterpart in the reference's operator (a mask tensor can hide keys, not
 * say that a query row is padding): when given, query rows i >= q_lens[b] are declared padding, their output
 * rows are unspecified (a kernel may skip them or compute them), and a caller that pads both sides of a
 * self-attention batch passes the same lengths here and in `kv_lens`.  Rows below the length are unaffected.
 *
 * Output dtype equals the input dtype; accumulation is f32
 * (crates/incin-backends/src/dtype_policy.rs:64-104).
 */
typedef struct {
    int32_t dtype;                 /* INCIN_ROCM_F32 / F16 / BF16: q, k, v, o and add_mask all share it */
    int32_t device;
    int64_t B, Hq, Hkv, Sq, Skv, D, Dv;
    int64_t q_stride[3];           /* elements: batch, head, sequence; the last axis has stride 1 */
    int64_t k_stride[3];
    int64_t v_stride[3];
    int64_t o_stride[3];
    const void* q;
    const void* k;
    const void* v;
    void* o;
    float scale;                   /* resolved by the caller: (float) scale.unwrap_or(1/sqrt(D)), the f64 -> f32
                                      cast of shape_ops.rs:1259-1261 + elementwise_kernel.rs:87 */
    int32_t causal;                /* 0 / 1 */
    const int32_t* kv_lens;        /* nullable device pointer, B entries */
    const void* add_mask;          /* nullable device pointer, dtype `dtype` */
    int64_t mask_stride[4];        /* elements: batch, query head, query row, key; 0 = broadcast */
    void* workspace;               /* device scratch for split-KV partials; see incin_rocm_sdpa_workspace */
    size_t workspace_bytes;
    int32_t num_splits;            /* splits of the key axis (split-KV kernels; 16-bit MFMA prefill kernel): 0 = library chooses, 1 = none */
    int32_t impl;                  /* INCIN_ROCM_IMPL_*; AUTO unless a test pins a kernel */
    const int32_t* q_lens;         /* nullable device pointer, B entries: rows at and beyond are padding */
    float* lse;                    /* nullable device pointer, contiguous f32 [B, Hq, Sq]: receives log sum_j exp(x_ij) of
                                      every row (natural log of the softmax normaliser; -inf for a row with no visible
                                      key) - what incin_rocm_sdpa_bwd needs from the forward.  Every kernel writes it
                                      (launches that split the key axis: their combine pass) */
} incin_rocm_sdpa_desc_t;

/* Validates the descriptor and reports the scratch bytes and the split count the
 * launch will use (0 bytes and 1 split when the chosen kernel needs none).
 * `impl_out` (nullable) receives the INCIN_ROCM_IMPL_* the library will run. */
int incin_rocm_sdpa_workspace(const incin_rocm_sdpa_desc_t* desc, size_t* bytes, int32_t* splits, int32_t* impl_out);

/* Enqueues the kernels on `stream` (NULL = the device's default stream) and
 * returns without waiting.  The library keeps no pointer after return except the
 * stream-ordered use of the buffers named in the descriptor, which the caller
 * keeps alive until the stream has been synchronised.
 *
 * Workspace.  Two kinds of launch need scratch memory, of the size incin_rocm_sdpa_workspace reports: launches that split
 * the key axis - the split-KV kernels, and the MFMA prefill kernels when few row blocks meet many keys - (partial
 * results of the splits) and the MFMA prefill kernels with a dense mask
 * (one byte per block of 32 query rows x 32 keys of the mask: which blocks it hides, which it leaves alone;
 * written by a small kernel of the same launch).  The contents need not survive the launch and
 * need no initialisation, but two launches that may run at the same time - other streams, other host threads, a
 * recorded graph replayed beside eager launches - must not be given the same workspace: they would overwrite
 * each other's partial results or block flags.  A recorded launch keeps using the workspace
 * it was recorded with on every replay. */
int incin_rocm_sdpa_fwd(const incin_rocm_sdpa_desc_t* desc, void* stream);

/* The same launch for callers that cannot allocate device memory (code under graph capture, serving loops and
 * harnesses that forbid it).  No counterpart in the reference.  `workspace` and `workspace_bytes` of the
 * descriptor are ignored: the scratch memory is a buffer of INCIN_ROCM_STATIC_SCRATCH_BYTES that is part of the
 * library's code object (one copy per device, held until the process ends), and the call makes no device or
 * host allocation.  A request whose scratch need (incin_rocm_sdpa_workspace) exceeds the buffer is refused with
 * INCIN_ROCM_EWORKSPACE.  Every call on a device shares that device's buffer: calls that may overlap in time on
 * one device race, so keep them on one stream or order them with events. */
#define INCIN_ROCM_STATIC_SCRATCH_BYTES (8u << 20)
int incin_rocm_sdpa_fwd_static(const incin_rocm_sdpa_desc_t* desc, void* stream);

/* ---- attention backward --------------------------------------------------------
 * The reference has no backward kernel for attention: its gradient is what walking the tape of the composed ops
 * gives (crates/incin-backends/src/cpu/ops/shape_ops.rs:1245-1269 records matmul, mul_scalar, add, log_softmax,
 * exp, matmul; crates/incin-backends/src/cpu/tape.rs:149-176 walks it).  This computes the same dq, dk, dv in
 * three launches from q, k, v, the forward's output o and row normalisers lse, and the upstream gradient d_o.
 *
 * `fwd` is the forward's descriptor as it was launched with `lse` set (o and lse are inputs here); causal,
 * kv_lens and the grouped-query layout carry over; d_k and d_v are summed over the query heads of a group.
 * Covered: f32 / f16 / bf16, D and Dv up to 256, dense additive mask, causal, kv_lens, q_lens (padding query rows: their
 * O, lse and d_o rows are never read, their d_q rows are written as zero and they add nothing to d_k and d_v).
 * fwd.impl picks the kernels: AUTO = matrix-core kernels where they apply - D and Dv up to 128 in whole 16-byte vectors (zero-padded
 * into instances for 64 and 128); f16 / bf16 with a positive scale, f32 (IEEE single-precision matrix instructions) with any finite
 * scale; both with 16-byte aligned rows, and a dense mask of non-negative strides of which 64 rows fit 32-bit byte offsets
 * - and generic f32-arithmetic kernels otherwise; GENERIC and MFMA pin one or the other.  A query row with no visible key (NaN in the forward) gets a zero gradient and
 * contributes nothing to d_k and d_v, where the reference's tape would spread NaN over the whole head.
 * The workspace holds two floats per query row (2 x [B, Hq, Sq]) and, for a dense mask on the matrix-core kernels, a byte
 * per 32 rows x 32 keys of the mask behind them, and for a call on the matrix-core kernels that does not fill the device
 * (f32; 16-bit storage with few KV heads) up to four f32 copies of the gradients' shapes, which workgroups that share a block
 * of rows or keys sum into (ask incin_rocm_sdpa_bwd_workspace for the size: it depends on the device's compute-unit count);
 * d_q, d_k, d_v are fully overwritten.
 * Streams: everything the call launches is ordered behind the work already on `stream` and ahead of whatever `stream` gets
 * next.  A call of the matrix-core kernels that is short of work may run its dQ kernel on a stream of the library's own
 * beside the dK/dV kernel (forked from and joined to `stream` with events; the library's streams have the default priority,
 * are created on demand, shared by all calls on a device and kept until the process ends).  Never while `stream` is being
 * captured into a graph, and never with INCIN_ROCM_BWD_STREAMS=1 in the environment (read at every call). */
typedef struct {
    incin_rocm_sdpa_desc_t fwd;
    const void* d_o;               /* [B, Hq, Sq, D], dtype of the operands */
    int64_t d_o_stride[3];
    void* d_q;                     /* [B, Hq, Sq, D] */
    int64_t d_q_stride[3];
    void* d_k;                     /* [B, Hkv, Skv, D] */
    int64_t d_k_stride[3];
    void* d_v;                     /* [B, Hkv, Skv, D] */
    int64_t d_v_stride[3];
    void* workspace;
    size_t workspace_bytes;
} incin_rocm_sdpa_bwd_desc_t;
size_t incin_rocm_sizeof_sdpa_bwd_desc(void);
int incin_rocm_sdpa_bwd_workspace(const incin_rocm_sdpa_bwd_desc_t* desc, size_t* bytes);
int incin_rocm_sdpa_bwd(const incin_rocm_sdpa_bwd_desc_t* desc, void* stream);

/* ---- diagnostics ------------------------------------------------------------------
 * No counterpart in the reference.  One launch of a loop of bf16 matrix instructions (v_mfma_f32_32x32x16_bf16, one
 * workgroup of two wavefronts per SIMD on every compute unit, `iterations` x 4 instructions per wavefront) whose operands
 * are whatever the 256 KiB at `operands` hold - zeros, random values, a slice of real inputs.  mix 0: matrix instructions
 * only; mix 1: with the vector and LDS instructions the prefill kernel issues per matrix instruction.  The rate a device
 * sustains depends on that data (its power management lowers the clock under the switching activity of random values),
 * and it is the ceiling the 16-bit attention kernels live under; bench.py reports it beside their roofline.
 * `sink` takes 2 KiB per compute unit.  *flops = FLOPs of the launch; time it with events on `stream`. */
int incin_rocm_matrix_rate(int32_t dev, const void* operands, void* sink, int32_t mix, int32_t iterations, double* flops, void* stream);

/* No counterpart in the reference.  One launch of a kernel that does nothing but read `bytes` bytes at `src` (a positive
 * multiple of 128 MiB) with 16-byte loads, marked non-temporal or not, and throw them away: the rate the memory system
 * delivers to a kernel that only reads, the ceiling the split-KV kernels live under; bench.py reports it beside their
 * roofline.  `sink` takes 16 KiB.  Time it with events on `stream`. */
int incin_rocm_read_rate(int32_t dev, const void* src, size_t bytes, int32_t nontemporal, void* sink, void* stream);

/* No counterpart in the reference.  One launch that writes `pattern` into every 32-bit word of the LDS of every compute
 * unit (1024 workgroups of 160 KiB).  The matrix-core kernels pad a head dimension below their instance's with zeros
 * that the copy engine writes into LDS, and read nothing else they have not written; a test fills LDS with the bit
 * pattern of a NaN first and shows that no result depends on what LDS held.  `sink` takes 4 bytes and is never written. */
int incin_rocm_lds_fill(int32_t dev, uint32_t pattern, void* sink, void* stream);

/* ---- key/value cache append ----------------------------------------------------
 * No counterpart in the reference (it has no cache: a decode loop there concatenates tensors,
 * TensorOps::cat, and re-runs the operator).  Copies S_new new key and value rows per (batch, kv head) into
 * preallocated caches [B, Hkv, S_max, D] / [.., Dv] at row kv_lens[b], then advances kv_lens[b] by S_new - all
 * on the device and stream-ordered, so that (append, incin_rocm_sdpa_fwd with the same kv_lens) is a decode step
 * that needs nothing from the host and can be recorded into a launch graph once and replayed per token.
 * Rows that would land at or beyond S_max are dropped and kv_lens saturates at S_max: the caller sizes the cache.
 * Strides are in elements (batch, head, row), the last axis has stride 1. */
typedef struct {
    int32_t dtype;                 /* INCIN_ROCM_F32 / F16 / BF16 */
    int32_t device;
    int64_t B, Hkv, S_new, S_max, D, Dv;
    const void* k_new;
    const void* v_new;
    int64_t k_new_stride[3];
    int64_t v_new_stride[3];
    void* k_cache;
    void* v_cache;
    int64_t k_cache_stride[3];
    int64_t v_cache_stride[3];
    int32_t* kv_lens;              /* device pointer, B entries, read and advanced */
} incin_rocm_kv_append_desc_t;
size_t incin_rocm_sizeof_kv_append_desc(void);
int incin_rocm_kv_append(const incin_rocm_kv_append_desc_t* desc, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* INCIN_ROCM_H */
