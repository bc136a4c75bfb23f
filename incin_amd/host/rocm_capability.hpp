// Host-side mirror of incin's capability registry for the `rocm` device, in C++ for the same reason as
// rocm_backend.hpp.  It stands where the ROCM_CAPABILITIES table and its registry() arm would stand in
// crates/incin-backends/src/capability.rs (:140-203, :339-352), resolves queries the way
// incin-core/src/exec/capability.rs:215-297 does (first rule that matches wins; the reason for a refusal is the
// first constraint no rule of the operation satisfied) and renders the per-device table the way
// crates/incin-backends/src/capability_docs.rs:129-170 does, so that "what this backend runs" is a table a
// planner can query and docs can be generated from - not a trait method that errors at run time.
//
// The reference's tables have no row for attention (its operator is a trait method); the mirror adds the
// operation kind `attention` - family `reduction`, like `matmul` (incin-core/src/shapes/error.rs:94-135) - and
// registers it for this device, plus the one row the CPU table would gain for its composed implementation
// (cpu/ops/shape_ops.rs:1245-1269).
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

namespace incin_rocm_host {
namespace capability {

constexpr int MAX_RANK = 8;      // incin-macros/src/rank.rs:25

// incin-core/src/shapes/error.rs:38-85, in declaration order, plus Attention
enum class OperationKind : int32_t {
    Storage, Fill, Random, Pointwise, Reduction, Normalization, Broadcast, Reshape, Flatten, Squeeze, Unsqueeze,
    Permute, Transpose, Slice, Concat, Stack, MatMul, Conv1d, Conv2d, Pool1d, Pool2d, AdaptiveAvgPool2d, Embedding,
    Attention,
    Count_
};
const char* name(OperationKind op);
OperationKind family(OperationKind op);

enum class DTypeId : int32_t { U8, U32, I64, BF16, F16, F32, F64, Q8_0, Count_ };
const char* name(DTypeId d);

// incin-core/src/exec/meta.rs:21-35
enum class LayoutClass : int32_t { Strided, Contiguous, ScalarLeft, ScalarRight, ContiguousLastAxis, RowWise, ChannelWise, Count_ };
const char* as_str(LayoutClass l);

enum class MathMode : int32_t { Precise, Fast, Count_ };      // incin-core/src/exec/policy.rs:20-24
const char* as_str(MathMode m);

enum class ImplementationKind : int32_t { Native, Composed, Fallback };
const char* name(ImplementationKind k);

enum class DeviceKind : int32_t { Cpu, Cuda, Wgpu, Metal, Rocm };
const char* name(DeviceKind d);

struct CapabilityQuery {
    OperationKind operation;
    DTypeId dtype;
    LayoutClass layout;
    int rank;
    bool training;
    MathMode math_mode;
};

struct UnsupportedReason {
    enum class Kind : int32_t { Operation, DType, Layout, Rank, Training, MathMode, MissingDeviceFeature } kind;
    OperationKind operation = OperationKind::Storage;
    DTypeId dtype = DTypeId::F32;
    LayoutClass layout = LayoutClass::Contiguous;
    int rank = 0, min = 0, max = 0;
    MathMode math_mode = MathMode::Precise;
    const char* feature = "";
    std::string to_string() const;          // the reference's Display text
};

struct SupportLevel {
    enum class Kind : int32_t { Native, Composed, Fallback, Unsupported } kind;
    UnsupportedReason reason{};              // meaningful when kind == Unsupported
    bool is_supported() const { return kind != Kind::Unsupported; }
    bool is_device_local() const { return kind == Kind::Native || kind == Kind::Composed; }
};

struct CapabilityRule {
    OperationKind operation;
    std::vector<DTypeId> dtypes;
    std::vector<LayoutClass> layouts;
    int min_rank, max_rank;
    bool training;
    std::vector<MathMode> math_modes;
    ImplementationKind implementation;
};

class CapabilityRegistry {
  public:
    explicit CapabilityRegistry(const std::vector<CapabilityRule>* rules) : rules_(rules) {}
    const std::vector<CapabilityRule>& registrations() const { return *rules_; }
    SupportLevel support(const CapabilityQuery& q) const;

  private:
    const std::vector<CapabilityRule>* rules_;
};

// What the rocm backend registers, and the row the CPU table gains.
const std::vector<CapabilityRule>& rocm_capabilities();
const std::vector<CapabilityRule>& cpu_attention_capabilities();
// Rocm: rocm_capabilities(); Cpu: only the attention row (the mirror does not restate the reference's own tables);
// every other device: no registrations.
CapabilityRegistry registry(DeviceKind device);
SupportLevel support(DeviceKind device, const CapabilityQuery& q);

// The "## `device`" section of docs/capabilities.md for a rule list (capability_docs.rs:129-154), and the
// element-types-by-operation table over several devices (capability_docs.rs:75-127).
std::string device_section(DeviceKind device, const std::vector<CapabilityRule>& rules);
std::string summary(const std::vector<std::pair<DeviceKind, const std::vector<CapabilityRule>*>>& devices);

}  // namespace capability
}  // namespace incin_rocm_host
