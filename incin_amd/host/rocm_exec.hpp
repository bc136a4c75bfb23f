// Operation descriptors and their executor for the rocm backend mirror: the part of incin's "validated
// descriptor -> Execute" path (incin-core/src/exec: ShapeRule::lower produces a Validated<Spec>, a backend
// implements Execute<Spec>; used by crates/incin-backends/src/external/conformance.rs:176-198,280-297) that
// attention needs.  AttentionSpec states as proven fields what the tensor-level operator can only receive as a
// mask tensor: causal alignment, per-batch key counts, the grouped-query layout, the scale.  lower_attention()
// is the shape rule (no device needed); execute() checks the handles it is given against the proof - arity,
// shapes, dtype: Validated proves shapes, not handles - and runs the operator.
#pragma once
#include <optional>
#include <vector>

#include "rocm_backend.hpp"

namespace incin_rocm_host {

struct AttentionSpec {
    std::vector<int64_t> q_dims, k_dims, v_dims;      // as given
    std::vector<int64_t> out_dims;                    // broadcast batch axes + [Sq, Dv]
    int64_t group = 1;                                // query heads per key/value head (last batch axis of q over 1 of k, v)
    bool causal = false;                              // query i sees keys j <= i + Skv - Sq
    std::optional<std::vector<int32_t>> kv_lens;      // keys j >= kv_lens[b] masked; one entry per index of the batch axis
    std::optional<std::vector<int32_t>> q_lens;       // query rows i >= q_lens[b] are padding: output rows unspecified
    std::optional<double> scale;                      // None: 1/sqrt(D)
    DType dtype = DType::F32;
};

struct ReshapeSpec {
    std::vector<int64_t> in_dims, out_dims;
};

// Shape rules.  Errors are ShapeMismatch with the operation's name, as the reference's rules report them.
Error lower_attention(const std::vector<int64_t>& q_dims, const std::vector<int64_t>& k_dims, const std::vector<int64_t>& v_dims,
                      DType dtype, bool causal, const std::optional<std::vector<int32_t>>& kv_lens, std::optional<double> scale,
                      AttentionSpec* out, const std::optional<std::vector<int32_t>>& q_lens = std::nullopt);
Error lower_reshape(const std::vector<int64_t>& in_dims, const std::vector<int64_t>& out_dims, ReshapeSpec* out);

// Executors: inputs are borrowed storages, the output is a new storage (attention) or a view (reshape).
Error execute(const AttentionSpec& spec, const std::vector<const RocmStorage*>& inputs, RocmStorage* out);
Error execute(const ReshapeSpec& spec, const std::vector<const RocmStorage*>& inputs, RocmStorage* out);

// ---- device detection (crates/incin-backends/src/detect.rs:26-95 with the rocm arm) ---------------------------
// kinds as capability::DeviceKind: 0 cpu, 1 cuda, 2 wgpu, 3 metal, 4 rocm
struct DeviceId {
    int32_t kind = 0;
    int32_t ordinal = 0;
};
bool is_compiled_in(int32_t kind);                         // this mirror holds the rocm backend only
std::optional<DeviceId> probe(int32_t kind);               // rocm: a device exists and memory can be allocated on it
DeviceId detect_device_in(const std::vector<int32_t>& preference);     // first kind that probes; cpu ends the chain
const std::vector<int32_t>& preference();                  // cuda, rocm, metal, wgpu, cpu

// ---- runtime dispatch (crates/incin-backends/src/dispatch.rs:54-66, 1196-1225 with the rocm arm) ---------------
// A storage that says which backend holds the data.  The reference's enum has one variant per compiled-in backend plus
// `Unavailable`; this mirror compiles in the rocm arm only, so the others never occur here.
struct DispatchStorage {
    enum class Holder { Unavailable, Rocm } holder = Holder::Unavailable;
    RocmStorage rocm;
    static DispatchStorage on_rocm(RocmStorage s);
};
struct DispatchBackend {
    // Routes to the backend that holds q, k and v; operands (or a mask) held elsewhere are an error, never a copy:
    // "mismatched backends in SDPA" / "mismatched mask backend", the reference's messages.
    static Error scaled_dot_product_attention(const DispatchStorage& q, const DispatchStorage& k, const DispatchStorage& v,
                                              const DispatchStorage* mask, std::optional<double> scale, DispatchStorage* out);
};

}  // namespace incin_rocm_host
