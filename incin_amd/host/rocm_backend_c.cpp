#include "rocm_backend_c.h"

#include <cstring>
#include <string>

#include "rocm_backend.hpp"
#include "rocm_capability.hpp"

using namespace incin_rocm_host;

struct incin_host_storage {
    RocmStorage s;
};

namespace {
thread_local std::string g_last_error;

int finish(const Error& e)
{
    if (e) g_last_error = e.message;
    return (int)e.kind;
}
int give(const Error& e, RocmStorage&& s, incin_host_storage** out)
{
    if (!e) *out = new incin_host_storage{std::move(s)};
    return finish(e);
}
}  // namespace

extern "C" {

const char* incin_host_last_error(void) { return g_last_error.c_str(); }

int incin_host_from_bytes(const void* bytes, size_t nbytes, const int64_t* dims, int32_t rank, int32_t dtype, int32_t device,
                          incin_host_storage** out)
{
    RocmStorage s;
    Error e = RocmBackend::from_bytes(bytes, nbytes, std::vector<int64_t>(dims, dims + rank), (DType)dtype, device, &s);
    return give(e, std::move(s), out);
}

int incin_host_numel(const incin_host_storage* s, int64_t* out) { *out = s->s.numel(); return 0; }
int incin_host_rank(const incin_host_storage* s, int32_t* out) { *out = (int32_t)s->s.shape.size(); return 0; }
int incin_host_shape(const incin_host_storage* s, int64_t* dims_out)
{
    for (size_t i = 0; i < s->s.shape.size(); ++i) dims_out[i] = s->s.shape[i];
    return 0;
}
int incin_host_dtype(const incin_host_storage* s, int32_t* out) { *out = (int32_t)s->s.dtype; return 0; }

int incin_host_to_bytes(const incin_host_storage* s, void* out, size_t capacity)
{
    std::vector<uint8_t> bytes;
    Error e = RocmBackend::to_bytes(s->s, &bytes);
    if (!e && bytes.size() > capacity) e = Error{ErrorKind::Msg, "to_bytes: destination too small"};
    if (!e && !bytes.empty()) std::memcpy(out, bytes.data(), bytes.size());
    return finish(e);
}

int incin_host_transpose(const incin_host_storage* s, int32_t a, int32_t b, incin_host_storage** out)
{
    RocmStorage r;
    Error e = RocmBackend::transpose(s->s, a, b, &r);
    return give(e, std::move(r), out);
}

int incin_host_broadcast_as(const incin_host_storage* s, const int64_t* dims, int32_t rank, incin_host_storage** out)
{
    RocmStorage r;
    Error e = RocmBackend::broadcast_as(s->s, std::vector<int64_t>(dims, dims + rank), &r);
    return give(e, std::move(r), out);
}

int incin_host_narrow(const incin_host_storage* s, int32_t dim, int64_t start, int64_t len, incin_host_storage** out)
{
    RocmStorage r;
    Error e = RocmBackend::narrow(s->s, dim, start, len, &r);
    return give(e, std::move(r), out);
}

int incin_host_tag_causal(const incin_host_storage* mask, incin_host_storage** out)
{
    RocmStorage r;
    Error e = RocmBackend::tag_causal(mask->s, &r);
    return give(e, std::move(r), out);
}

int incin_host_tag_key_padding(const incin_host_storage* mask, const int32_t* lens, int64_t count, incin_host_storage** out)
{
    RocmStorage r;
    Error e = RocmBackend::tag_key_padding(mask->s, std::vector<int32_t>(lens, lens + count), &r);
    return give(e, std::move(r), out);
}

int incin_host_scaled_dot_product_attention(const incin_host_storage* q, const incin_host_storage* k, const incin_host_storage* v,
                                            const incin_host_storage* mask, int32_t has_scale, double scale,
                                            incin_host_storage** out)
{
    RocmStorage r;
    Error e = RocmBackend::scaled_dot_product_attention(q->s, k->s, v->s, mask ? &mask->s : nullptr,
                                                        has_scale ? std::optional<double>(scale) : std::nullopt, &r);
    return give(e, std::move(r), out);
}

void incin_host_release(incin_host_storage* s) { delete s; }

int64_t incin_host_last_launch_count(void) { return incin_rocm_host::last_launch_count(); }


// ---- capability registry ------------------------------------------------------------------------------------
namespace cap = incin_rocm_host::capability;

const char* incin_host_capability_name(int32_t what, int32_t value)
{
    switch (what) {
        case 0: return cap::name((cap::OperationKind)value);
        case 1: return cap::name((cap::DTypeId)value);
        case 2: return cap::as_str((cap::LayoutClass)value);
        case 3: return cap::as_str((cap::MathMode)value);
        case 4: return cap::name((cap::ImplementationKind)value);
        case 5: return value >= 0 && value <= 4 ? cap::name((cap::DeviceKind)value) : "?";
        default: return "?";
    }
}

int32_t incin_host_capability_max_rank(void) { return cap::MAX_RANK; }

int incin_host_capability_support(int32_t device_kind, int32_t operation, int32_t dtype, int32_t layout, int32_t rank,
                                  int32_t training, int32_t math_mode, int32_t* reason_kind, char* reason, size_t capacity)
{
    cap::CapabilityQuery q{(cap::OperationKind)operation, (cap::DTypeId)dtype, (cap::LayoutClass)layout, rank, training != 0,
                           (cap::MathMode)math_mode};
    const cap::SupportLevel lv = cap::support((cap::DeviceKind)device_kind, q);
    if (!lv.is_supported()) {
        if (reason_kind) *reason_kind = (int32_t)lv.reason.kind;
        if (reason && capacity) {
            const std::string text = lv.reason.to_string();
            const size_t n = text.size() < capacity - 1 ? text.size() : capacity - 1;
            std::memcpy(reason, text.data(), n);
            reason[n] = 0;
        }
    }
    return (int)lv.kind;
}

int32_t incin_host_capability_rule_count(int32_t device_kind)
{
    return (int32_t)cap::registry((cap::DeviceKind)device_kind).registrations().size();
}

int incin_host_capability_rule(int32_t device_kind, int32_t index, int32_t* operation, uint32_t* dtypes, uint32_t* layouts,
                               int32_t* min_rank, int32_t* max_rank, int32_t* training, uint32_t* math_modes,
                               int32_t* implementation)
{
    const std::vector<cap::CapabilityRule>& rules = cap::registry((cap::DeviceKind)device_kind).registrations();
    if (index < 0 || (size_t)index >= rules.size()) return finish(Error{ErrorKind::Msg, "capability rule index out of range"});
    const cap::CapabilityRule& r = rules[index];
    *operation = (int32_t)r.operation;
    *dtypes = *layouts = *math_modes = 0;
    for (cap::DTypeId d : r.dtypes) *dtypes |= 1u << (int)d;
    for (cap::LayoutClass l : r.layouts) *layouts |= 1u << (int)l;
    for (cap::MathMode m : r.math_modes) *math_modes |= 1u << (int)m;
    *min_rank = r.min_rank;
    *max_rank = r.max_rank;
    *training = r.training ? 1 : 0;
    *implementation = (int32_t)r.implementation;
    return 0;
}

size_t incin_host_capability_docs(char* out, size_t capacity)
{
    const std::string text = cap::summary({{cap::DeviceKind::Cpu, &cap::cpu_attention_capabilities()},
                                           {cap::DeviceKind::Rocm, &cap::rocm_capabilities()}}) +
                             cap::device_section(cap::DeviceKind::Cpu, cap::cpu_attention_capabilities()) +
                             cap::device_section(cap::DeviceKind::Rocm, cap::rocm_capabilities());
    if (out && capacity) {
        const size_t n = text.size() < capacity - 1 ? text.size() : capacity - 1;
        std::memcpy(out, text.data(), n);
        out[n] = 0;
    }
    return text.size();
}

}  // extern "C"
