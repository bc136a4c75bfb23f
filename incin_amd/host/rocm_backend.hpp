// Host-side mirror of the part of incin's backend interface that the attention path uses, written
// in C++ because no Rust toolchain exists in this build pipeline.  It stands where
// crates/incin-backends/src/rocm/{storage,backend}.rs would stand: storage with shape / strides /
// dtype / device (cf. cuda/storage.rs:24-59, cpu/storage.rs:199-204), byte round trips
// (Backend::from_bytes / to_bytes, cuda/backend.rs:1905-1937), metadata-only views
// (cpu/storage.rs:308-325) and TensorOps::scaled_dot_product_attention
// (incin-core/src/tensor/backend.rs:485-492) with the reference's argument meaning and error kinds
// (incin-core/src/err.rs:109-223).  All device work goes through the C ABI in include/incin_rocm.h.
#pragma once
#include <cstddef>
#include <cstdint>
#include <memory>
#include <optional>
#include <string>
#include <vector>

namespace incin_rocm_host {

enum class DType : int32_t { F32 = 0, F16 = 1, BF16 = 2 };
inline size_t dtype_size(DType d) { return d == DType::F32 ? 4 : 2; }

// The variants of incin_core::Error this path can produce.
enum class ErrorKind : int32_t {
    None = 0,
    Msg = 1,
    ShapeMismatch = 2,
    DTypeStorageMismatch = 3,
    DeviceMismatch = 4,
    UnsupportedDType = 5,
    InvalidDeviceOrdinal = 6,
    OutOfMemory = 7,
    UnsupportedBackendOperation = 8,
};

struct Error {
    ErrorKind kind = ErrorKind::None;
    std::string message;
    explicit operator bool() const { return kind != ErrorKind::None; }
};

// One device allocation, released when the last storage that views it goes away.  Released, not freed: the buffer goes back
// to a pool per device, stamped with an event on the stream the releasing thread works on, and is handed out again to
// that same stream at once (its work is ordered behind what still uses the buffer) or to another stream once the event
// has passed - the stream-ordered lifetime the reference's CUDA buffers have (cuda/storage.rs:171-177, 225-233).  So an
// operator can drop temporaries and workspaces that its kernels are still using without waiting for the device.
class RocmBuffer {
  public:
    RocmBuffer(int32_t device, void* ptr, size_t bytes) : device_(device), ptr_(ptr), bytes_(bytes) {}
    ~RocmBuffer();
    RocmBuffer(const RocmBuffer&) = delete;
    RocmBuffer& operator=(const RocmBuffer&) = delete;
    void* ptr() const { return ptr_; }
    size_t bytes() const { return bytes_; }
    int32_t device() const { return device_; }

  private:
    int32_t device_;
    void* ptr_;
    size_t bytes_;
};

// What a mask storage may declare about its contents so the backend need not read them.
struct MaskTag {
    enum Kind { Causal, KeyPadding, CausalKeyPadding } kind;      // (the last: the sum of the two masks)
    std::shared_ptr<RocmBuffer> lens;      // KeyPadding, CausalKeyPadding: int32 key counts, one per batch entry
    int64_t lens_count = 0;
};

struct RocmStorage {
    std::shared_ptr<RocmBuffer> buffer;
    std::vector<int64_t> shape;
    std::vector<int64_t> strides;          // elements; 0 on a broadcast axis
    int64_t offset_elements = 0;
    DType dtype = DType::F32;
    int32_t device = 0;
    std::optional<MaskTag> mask_tag;

    int64_t numel() const;
    bool is_contiguous() const;
    const char* data() const { return static_cast<const char*>(buffer->ptr()) + offset_elements * (int64_t)dtype_size(dtype); }
};

// What a recording (launch graph) keeps alive: buffers released while it was being recorded - the recorded kernels use
// them at every replay.  They return to the pool when the recording is destroyed.
struct RecordedGraph {
    void* graph = nullptr;        // incin_rocm_graph_* handle
    int32_t device = 0;
    std::vector<std::pair<void*, size_t>> retained;
    ~RecordedGraph();
    RecordedGraph() = default;
    RecordedGraph(const RecordedGraph&) = delete;
    RecordedGraph& operator=(const RecordedGraph&) = delete;
};

struct RocmBackend {
    // The stream the calling thread's operators launch on and its buffers are ordered by (nullptr: the device's default
    // stream, as the reference's backends use: cuda/ops/matmul.rs:57-90).  to_bytes waits for it.
    static void set_stream(void* stream);
    static void* stream();
    // Recording of the calling thread's work on its stream (not the default stream) into a launch graph.  While recording,
    // nothing may be allocated from or returned to the device: buffers come from the pool (run the same operators once
    // beforehand: what they released is what the recording finds there) and released ones are kept with the recording.
    static Error begin_recording(int32_t device);
    static Error end_recording(std::unique_ptr<RecordedGraph>* out);
    static Error replay(const RecordedGraph& g);
    // Pool counters of a device (for tests): device allocations made so far, buffers handed out from the pool, bytes idle
    // in the pool.  trim_pool waits for the device and frees what is idle.
    struct PoolStats { int64_t device_allocs = 0, reused = 0, idle_bytes = 0; };
    static PoolStats pool_stats(int32_t device);
    static Error trim_pool(int32_t device);

    // Backend::from_bytes: one allocation + one host-to-device copy; row-major contiguous.
    static Error from_bytes(const void* bytes, size_t nbytes, const std::vector<int64_t>& dims, DType dtype, int32_t device,
                            RocmStorage* out);
    // Backend::to_bytes: logical (row-major) contents of the view.
    static Error to_bytes(const RocmStorage& s, std::vector<uint8_t>* out);
    static std::vector<int64_t> shape(const RocmStorage& s) { return s.shape; }

    // A dense row-major copy of a view (the same storage when it already is dense): CpuStorage::contiguous,
    // cpu/storage.rs:407-440.
    static Error contiguous(const RocmStorage& s, RocmStorage* out);

    // Metadata-only views, as the reference's storages provide.
    static Error transpose(const RocmStorage& s, int a, int b, RocmStorage* out);
    static Error broadcast_as(const RocmStorage& s, const std::vector<int64_t>& dims, RocmStorage* out);
    static Error narrow(const RocmStorage& s, int dim, int64_t start, int64_t len, RocmStorage* out);

    // Declarations about a mask's contents (the caller vouches for them): `tag_causal` says the storage holds
    // full(-inf).triu(1 + Skv - Sq) over its last two axes; `tag_key_padding` says it holds 0 for keys j < lens[b]
    // and -inf for the rest, constant over query rows and heads.
    static Error tag_causal(const RocmStorage& mask, RocmStorage* out);
    static Error tag_key_padding(const RocmStorage& mask, const std::vector<int32_t>& lens, RocmStorage* out);
    // The same declarations read off the mask's contents.  The reference's operator knows a mask only as a tensor
    // (cpu/ops/shape_ops.rs:1262-1266), and its callers build the causal mask as full(-inf).triu(1), key padding as 0 / -inf
    // per key and add the two: every row of such a mask is n zeros followed by -inf.  This reads the mask once on the
    // device (incin_rocm_mask_row_limits), waits for the result - the one synchronisation, which is why it is a call of its
    // own and not part of the operator: a backend makes it where the mask is made, once per mask - and tags `out` as
    // Causal, KeyPadding (one count per index of the first axis) or both, if that is what the rows say: *kind 0 none (out is
    // the mask untouched: values, holes, a window, counts the tag could not hold), 1 causal, 2 key padding, 3 both.  A tagged
    // mask runs on the facts in the forward and - where a mask tensor would send the gradients to the generic kernels -
    // in the backward.  Masks of rank 2 to 4.
    static Error infer_mask_tag(const RocmStorage& mask, RocmStorage* out, int* kind);

    // TensorOps::scaled_dot_product_attention.
    static Error scaled_dot_product_attention(const RocmStorage& q, const RocmStorage& k, const RocmStorage& v,
                                              const RocmStorage* mask, std::optional<double> scale, RocmStorage* out);

    // The same operator with what a descriptor states about masking (rocm_exec.hpp) instead of, or on top of, a mask
    // storage: causal alignment and per-batch key counts; both may hold at once.
    struct MaskFacts {
        bool causal = false;
        std::shared_ptr<RocmBuffer> kv_lens;      // int32 key counts on the device, one per batch entry
        int64_t kv_lens_count = 0;
        std::shared_ptr<RocmBuffer> q_lens;       // int32 query counts: rows at and beyond are padding, their output unspecified
        int64_t q_lens_count = 0;
    };
    static Error attention(const RocmStorage& q, const RocmStorage& k, const RocmStorage& v, const RocmStorage* mask,
                           std::optional<double> scale, const MaskFacts& facts, RocmStorage* out);

    // Gradients of the operator for an upstream gradient of the output's shape: the forward is run once more keeping its
    // row normalisers, then one backward call per forward launch.  The reference gets these by walking its tape of the
    // composed ops (cpu/tape.rs:149-176); like there, the mask is a constant.  dq, dk, dv are fresh contiguous storages of
    // the operands' shapes.  Keys and values shared by a group of query heads get the sum over the group from the kernels;
    // an operand broadcast along any other batch axis (or a query row repeated under a mask of several rows) gets its
    // gradient at the launches' shape first and the sum over the repetitions after (cpu/tape.rs:243-265); the upstream
    // gradient may be any view.  q_lens together with gradients is UnsupportedBackendOperation.
    struct AttentionGrads {
        RocmStorage dq, dk, dv;
    };
    static Error attention_backward(const RocmStorage& q, const RocmStorage& k, const RocmStorage& v, const RocmStorage* mask,
                                    std::optional<double> scale, const MaskFacts& facts, const RocmStorage& grad_out,
                                    RocmStorage* out, AttentionGrads* grads);

    // Reinterpret a contiguous storage under another shape of the same element count (metadata only).
    static Error reshape(const RocmStorage& s, const std::vector<int64_t>& dims, RocmStorage* out);
    // int32 values on the device (key counts of a descriptor).
    static Error upload_i32(const std::vector<int32_t>& values, int32_t device, std::shared_ptr<RocmBuffer>* out);

private:
    static Error attention_impl(const RocmStorage& q, const RocmStorage& k, const RocmStorage& v, const RocmStorage* mask,
                                std::optional<double> scale, const MaskFacts& facts, const RocmStorage* grad_out, RocmStorage* out,
                                AttentionGrads* grads);
};

// NumPy-style right-aligned broadcast of two shapes (cpu/stride.rs:86-106).
Error broadcast_shape(const std::vector<int64_t>& a, const std::vector<int64_t>& b, std::vector<int64_t>* out);

// Number of C-ABI attention calls the last scaled_dot_product_attention on this thread needed (1 unless batch
// axes could not be collapsed into the descriptor's batch / head strides).
int64_t last_launch_count();

}  // namespace incin_rocm_host
