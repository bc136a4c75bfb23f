#include "rocm_capability.hpp"

#include <algorithm>
#include <utility>

namespace incin_rocm_host {
namespace capability {

const char* name(OperationKind op)
{
    static const char* const names[] = {"storage", "fill", "random", "pointwise", "reduction", "normalization", "broadcast",
                                        "reshape", "flatten", "squeeze", "unsqueeze", "permute", "transpose", "slice",
                                        "concat", "stack", "matmul", "conv1d", "conv2d", "pool1d", "pool2d",
                                        "adaptive_avg_pool2d", "embedding", "attention"};
    const int i = (int)op;
    return i >= 0 && i < (int)OperationKind::Count_ ? names[i] : "?";
}

// Operations that only move or re-address bytes resolve dtype policy as `storage`; operations that sum many
// values into one as `reduction` - attention is two matrix products and a softmax, so it goes with matmul.
OperationKind family(OperationKind op)
{
    switch (op) {
        case OperationKind::Storage: case OperationKind::Broadcast: case OperationKind::Reshape: case OperationKind::Flatten:
        case OperationKind::Squeeze: case OperationKind::Unsqueeze: case OperationKind::Permute: case OperationKind::Transpose:
        case OperationKind::Slice: case OperationKind::Concat: case OperationKind::Stack: case OperationKind::Embedding:
            return OperationKind::Storage;
        case OperationKind::Fill: return OperationKind::Fill;
        case OperationKind::Random: return OperationKind::Random;
        case OperationKind::Pointwise: return OperationKind::Pointwise;
        case OperationKind::Normalization: return OperationKind::Normalization;
        default: return OperationKind::Reduction;
    }
}

const char* name(DTypeId d)
{
    static const char* const names[] = {"u8", "u32", "i64", "bf16", "f16", "f32", "f64", "q8_0"};
    const int i = (int)d;
    return i >= 0 && i < (int)DTypeId::Count_ ? names[i] : "?";
}

const char* as_str(LayoutClass l)
{
    static const char* const names[] = {"strided", "contiguous", "scalar-left", "scalar-right", "contiguous-last-axis",
                                        "row-wise", "channel-wise"};
    const int i = (int)l;
    return i >= 0 && i < (int)LayoutClass::Count_ ? names[i] : "?";
}

const char* as_str(MathMode m) { return m == MathMode::Precise ? "precise" : "fast"; }

const char* name(ImplementationKind k)
{
    return k == ImplementationKind::Native ? "native" : k == ImplementationKind::Composed ? "composed" : "fallback";
}

const char* name(DeviceKind d)
{
    static const char* const names[] = {"cpu", "cuda", "wgpu", "metal", "rocm"};
    return names[(int)d];
}

std::string UnsupportedReason::to_string() const
{
    const std::string op = name(operation);
    switch (kind) {
        case Kind::Operation: return "operation " + op + " is not registered";
        case Kind::DType: {
            // the reference prints the variant's Debug spelling here (U8, BF16, Q8_0, ...)
            std::string up = name(dtype);
            std::transform(up.begin(), up.end(), up.begin(), [](unsigned char c) { return (char)std::toupper(c); });
            return "dtype " + up + " is unsupported for " + op;
        }
        case Kind::Layout: return std::string("layout ") + as_str(layout) + " is unsupported for " + op;
        case Kind::Rank:
            return "rank " + std::to_string(rank) + " is unsupported for " + op + "; expected " + std::to_string(min) + "..=" +
                   std::to_string(max);
        case Kind::Training: return "training is unsupported for " + op;
        case Kind::MathMode: return std::string("math mode ") + as_str(math_mode) + " is unsupported for " + op;
        case Kind::MissingDeviceFeature: return std::string("required device feature ") + feature + " is unavailable";
    }
    return "";
}

namespace {
template <typename T> bool has(const std::vector<T>& v, T x) { return std::find(v.begin(), v.end(), x) != v.end(); }
}  // namespace

SupportLevel CapabilityRegistry::support(const CapabilityQuery& q) const
{
    // a query for an operation with registrations of its own is answered by those; otherwise by its family's
    bool exact = false;
    for (const CapabilityRule& r : *rules_) exact = exact || r.operation == q.operation;
    const OperationKind wanted = exact ? q.operation : family(q.operation);

    // how far down the list of constraints any rule of the operation got
    enum Stage { None, Op, DType, Layout, Rank, Training } reached = None;
    const CapabilityRule* rank_rule = nullptr;      // first rule that fits up to the layout: its bounds go into a rank refusal
    for (const CapabilityRule& r : *rules_) {
        if (r.operation != wanted) continue;
        Stage s = Op;
        if (has(r.dtypes, q.dtype)) {
            s = DType;
            if (has(r.layouts, q.layout)) {
                s = Layout;
                if (!rank_rule) rank_rule = &r;
                if (q.rank >= r.min_rank && q.rank <= r.max_rank) {
                    s = Rank;
                    if (!q.training || r.training) {
                        s = Training;
                        if (has(r.math_modes, q.math_mode)) {
                            SupportLevel ok;
                            ok.kind = r.implementation == ImplementationKind::Native     ? SupportLevel::Kind::Native
                                      : r.implementation == ImplementationKind::Composed ? SupportLevel::Kind::Composed
                                                                                         : SupportLevel::Kind::Fallback;
                            return ok;
                        }
                    }
                }
            }
        }
        reached = std::max(reached, s);
    }

    SupportLevel no;
    no.kind = SupportLevel::Kind::Unsupported;
    UnsupportedReason& why = no.reason;
    why.operation = q.operation;
    switch (reached) {
        case None: why.kind = UnsupportedReason::Kind::Operation; break;
        case Op: why.kind = UnsupportedReason::Kind::DType; why.dtype = q.dtype; break;
        case DType: why.kind = UnsupportedReason::Kind::Layout; why.layout = q.layout; break;
        case Layout:
            why.kind = UnsupportedReason::Kind::Rank;
            why.rank = q.rank;
            why.min = rank_rule->min_rank;
            why.max = rank_rule->max_rank;
            break;
        case Rank: why.kind = UnsupportedReason::Kind::Training; break;
        case Training: why.kind = UnsupportedReason::Kind::MathMode; why.math_mode = q.math_mode; break;
    }
    return no;
}

namespace {
const std::vector<DTypeId> ROCM_DTYPES = {DTypeId::BF16, DTypeId::F16, DTypeId::F32};      // what RocmStorage holds
const std::vector<MathMode> PRECISE = {MathMode::Precise};
const std::vector<LayoutClass> ANY_VIEW = {LayoutClass::Contiguous, LayoutClass::Strided, LayoutClass::RowWise};
// the attention kernels read q, k, v through their strides with the last axis dense: contiguous tensors and views
// whose rows are contiguous (transposes of batch axes, narrows, broadcasts)
const std::vector<LayoutClass> ROW_VIEWS = {LayoutClass::Contiguous, LayoutClass::RowWise};
}  // namespace

const std::vector<CapabilityRule>& rocm_capabilities()
{
    static const std::vector<CapabilityRule> rules = {
        // from_bytes / to_bytes: to_bytes gathers any view, from_bytes creates contiguous storage
        {OperationKind::Storage, ROCM_DTYPES, ANY_VIEW, 0, MAX_RANK, false, PRECISE, ImplementationKind::Native},
        // metadata-only views: transpose / narrow answer through the `storage` family, broadcast_as and reshape by rules of
        // their own
        {OperationKind::Broadcast, ROCM_DTYPES, ANY_VIEW, 0, MAX_RANK, false, PRECISE, ImplementationKind::Native},
        // reshape re-addresses contiguous storage; any other view is first gathered into a dense copy, as the reference's
        // reshape does (cpu/storage.rs:407-440)
        {OperationKind::Reshape, ROCM_DTYPES, {LayoutClass::Contiguous}, 0, MAX_RANK, false, PRECISE, ImplementationKind::Native},
        {OperationKind::Reshape, ROCM_DTYPES, {LayoutClass::Strided, LayoutClass::RowWise}, 0, MAX_RANK, false, PRECISE,
         ImplementationKind::Composed},
        // scaled_dot_product_attention and its gradients (RocmBackend::attention_backward): operands repeated along batch
        // axes get the sum of their repetitions' gradients, a mask may widen the scores, the upstream gradient may be any
        // view.  Outside what a query can say, the operator refuses head dimensions above 256 and gradients together with
        // query lengths (a descriptor field the reference's operator does not have).
        {OperationKind::Attention, ROCM_DTYPES, ROW_VIEWS, 2, MAX_RANK, true, PRECISE, ImplementationKind::Native},
        // operands whose last axis is strided (a transposed view): gathered into dense temporaries, then the same kernels
        {OperationKind::Attention, ROCM_DTYPES, {LayoutClass::Strided}, 2, MAX_RANK, true, PRECISE, ImplementationKind::Composed},
    };
    return rules;
}

const std::vector<CapabilityRule>& cpu_attention_capabilities()
{
    // the CPU operator is a composition of matmul, scalar multiply, add and softmax over f32 storage, recorded on
    // the autograd tape node by node (cpu/ops/shape_ops.rs:1245-1269): f32, any view, trainable, composed
    static const std::vector<CapabilityRule> rules = {
        {OperationKind::Attention, {DTypeId::F32}, {LayoutClass::Contiguous, LayoutClass::Strided}, 2, MAX_RANK, true, PRECISE,
         ImplementationKind::Composed},
    };
    return rules;
}

CapabilityRegistry registry(DeviceKind device)
{
    static const std::vector<CapabilityRule> none;
    switch (device) {
        case DeviceKind::Rocm: return CapabilityRegistry(&rocm_capabilities());
        case DeviceKind::Cpu: return CapabilityRegistry(&cpu_attention_capabilities());
        default: return CapabilityRegistry(&none);
    }
}

SupportLevel support(DeviceKind device, const CapabilityQuery& q) { return registry(device).support(q); }

namespace {
template <typename It, typename F> std::string join_code(It first, It last, F spell)
{
    std::string out;
    for (It it = first; it != last; ++it) {
        if (it != first) out += ", ";
        out += "`";
        out += spell(*it);
        out += "`";
    }
    return out;
}

std::string rank_range(const CapabilityRule& r)
{
    if (r.min_rank == 0 && r.max_rank == MAX_RANK) return "any";
    if (r.max_rank == MAX_RANK) return std::to_string(r.min_rank) + "+";
    if (r.min_rank == r.max_rank) return std::to_string(r.min_rank);
    return std::to_string(r.min_rank) + "\xe2\x80\x93" + std::to_string(r.max_rank);      // en dash
}
}  // namespace

std::string device_section(DeviceKind device, const std::vector<CapabilityRule>& rules)
{
    std::string out = std::string("## `") + name(device) + "`\n\n";
    if (rules.empty()) return out + "No registrations.\n\n";
    out += "| Operation | Element types | Layouts | Rank | Training | Implementation |\n";
    out += "|---|---|---|---|:--:|---|\n";
    for (const CapabilityRule& r : rules) {
        out += std::string("| `") + name(r.operation) + "` | ";
        out += join_code(r.dtypes.begin(), r.dtypes.end(), [](DTypeId d) { return name(d); }) + " | ";
        out += join_code(r.layouts.begin(), r.layouts.end(), [](LayoutClass l) { return as_str(l); }) + " | ";
        out += rank_range(r) + " | " + (r.training ? "yes" : "no") + " | " + name(r.implementation) + " |\n";
    }
    return out + "\n";
}

std::string summary(const std::vector<std::pair<DeviceKind, const std::vector<CapabilityRule>*>>& devices)
{
    std::vector<OperationKind> ops;
    for (const auto& d : devices)
        for (const CapabilityRule& r : *d.second)
            if (!has(ops, r.operation)) ops.push_back(r.operation);
    std::sort(ops.begin(), ops.end(), [](OperationKind a, OperationKind b) { return std::string(name(a)) < name(b); });

    std::string out = "## Element types by operation and backend\n\n| Operation |";
    for (const auto& d : devices) out += std::string(" ") + name(d.first) + " |";
    out += "\n|---|";
    for (size_t i = 0; i < devices.size(); ++i) out += "---|";
    out += "\n";
    for (OperationKind op : ops) {
        out += std::string("| `") + name(op) + "` |";
        for (const auto& d : devices) {
            std::vector<DTypeId> dtypes;      // union over the device's rules for this operation, first-seen order
            for (const CapabilityRule& r : *d.second)
                if (r.operation == op)
                    for (DTypeId t : r.dtypes)
                        if (!has(dtypes, t)) dtypes.push_back(t);
            if (dtypes.empty()) out += " \xe2\x80\x94 |";      // em dash: not registered
            else out += " " + join_code(dtypes.begin(), dtypes.end(), [](DTypeId t) { return name(t); }) + " |";
        }
        out += "\n";
    }
    return out + "\n";
}

}  // namespace capability
}  // namespace incin_rocm_host
