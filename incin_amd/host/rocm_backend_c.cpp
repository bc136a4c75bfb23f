#include "rocm_backend_c.h"

#include <cstring>
#include <memory>
#include <string>

#include "rocm_backend.hpp"
#include "rocm_capability.hpp"
#include "rocm_exec.hpp"

using namespace incin_rocm_host;

struct incin_host_storage {
    RocmStorage s;
};
struct incin_host_graph {
    std::unique_ptr<RecordedGraph> g;
};
struct incin_host_attention_spec {
    AttentionSpec spec;
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
int incin_host_strides(const incin_host_storage* s, int64_t* strides_out)
{
    for (size_t i = 0; i < s->s.strides.size(); ++i) strides_out[i] = s->s.strides[i];
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

int incin_host_infer_mask_tag(const incin_host_storage* mask, int32_t* kind, incin_host_storage** out)
{
    RocmStorage r;
    int k = 0;
    Error e = RocmBackend::infer_mask_tag(mask->s, &r, &k);
    if (kind) *kind = k;
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

int incin_host_attention_backward(const incin_host_storage* q, const incin_host_storage* k, const incin_host_storage* v,
                                  const incin_host_storage* mask, int32_t has_scale, double scale, const incin_host_storage* grad_out,
                                  incin_host_storage** out, incin_host_storage** dq, incin_host_storage** dk, incin_host_storage** dv)
{
    RocmStorage r;
    RocmBackend::AttentionGrads g;
    Error e = RocmBackend::attention_backward(q->s, k->s, v->s, mask ? &mask->s : nullptr,
                                              has_scale ? std::optional<double>(scale) : std::nullopt, RocmBackend::MaskFacts{},
                                              grad_out->s, &r, &g);
    if (e) return give(e, std::move(r), out);
    give(e, std::move(g.dq), dq);
    give(e, std::move(g.dk), dk);
    give(e, std::move(g.dv), dv);
    return give(e, std::move(r), out);
}

void incin_host_release(incin_host_storage* s) { delete s; }

int incin_host_data_ptr(const incin_host_storage* s, void** out) { *out = const_cast<char*>(s->s.data()); return 0; }
void incin_host_set_stream(void* stream) { RocmBackend::set_stream(stream); }
int incin_host_begin_recording(int32_t device) { return finish(RocmBackend::begin_recording(device)); }
int incin_host_end_recording(incin_host_graph** out)
{
    std::unique_ptr<RecordedGraph> g;
    Error e = RocmBackend::end_recording(&g);
    if (!e) *out = new incin_host_graph{std::move(g)};
    return finish(e);
}
int incin_host_replay(const incin_host_graph* g) { return finish(RocmBackend::replay(*g->g)); }
void incin_host_release_graph(incin_host_graph* g) { delete g; }
int incin_host_pool_stats(int32_t device, int64_t* device_allocs, int64_t* reused, int64_t* idle_bytes)
{
    const RocmBackend::PoolStats s = RocmBackend::pool_stats(device);
    *device_allocs = s.device_allocs;
    *reused = s.reused;
    *idle_bytes = s.idle_bytes;
    return 0;
}
int incin_host_trim_pool(int32_t device) { return finish(RocmBackend::trim_pool(device)); }

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


// ---- descriptors, detection ----------------------------------------------------------------------
int incin_host_lower_attention(const int64_t* q_dims, int32_t q_rank, const int64_t* k_dims, int32_t k_rank, const int64_t* v_dims,
                               int32_t v_rank, int32_t dtype, int32_t causal, const int32_t* kv_lens, int64_t kv_lens_count,
                               int32_t has_scale, double scale, const int32_t* q_lens, int64_t q_lens_count,
                               incin_host_attention_spec** out)
{
    std::optional<std::vector<int32_t>> lens, qlens;
    if (kv_lens_count >= 0) lens = std::vector<int32_t>(kv_lens, kv_lens + kv_lens_count);
    if (q_lens_count >= 0) qlens = std::vector<int32_t>(q_lens, q_lens + q_lens_count);
    AttentionSpec spec;
    Error e = lower_attention(std::vector<int64_t>(q_dims, q_dims + q_rank), std::vector<int64_t>(k_dims, k_dims + k_rank),
                              std::vector<int64_t>(v_dims, v_dims + v_rank), (DType)dtype, causal != 0, lens,
                              has_scale ? std::optional<double>(scale) : std::nullopt, &spec, qlens);
    if (!e) *out = new incin_host_attention_spec{std::move(spec)};
    return finish(e);
}

int incin_host_attention_spec_out_dims(const incin_host_attention_spec* spec, int64_t* dims_out, int32_t* rank_out, int64_t* group_out)
{
    for (size_t i = 0; i < spec->spec.out_dims.size(); ++i) dims_out[i] = spec->spec.out_dims[i];
    *rank_out = (int32_t)spec->spec.out_dims.size();
    if (group_out) *group_out = spec->spec.group;
    return 0;
}

int incin_host_execute_attention(const incin_host_attention_spec* spec, const incin_host_storage* const* inputs, int32_t n_inputs,
                                 incin_host_storage** out)
{
    std::vector<const RocmStorage*> in;
    for (int32_t i = 0; i < n_inputs; ++i) in.push_back(&inputs[i]->s);
    RocmStorage o;
    Error e = execute(spec->spec, in, &o);
    return give(e, std::move(o), out);
}

void incin_host_release_attention_spec(incin_host_attention_spec* spec) { delete spec; }

int incin_host_reshape(const incin_host_storage* s, const int64_t* dims, int32_t rank, incin_host_storage** out)
{
    RocmStorage o;
    Error e = RocmBackend::reshape(s->s, std::vector<int64_t>(dims, dims + rank), &o);
    return give(e, std::move(o), out);
}

int32_t incin_host_is_compiled_in(int32_t kind) { return is_compiled_in(kind) ? 1 : 0; }

int32_t incin_host_probe(int32_t kind)
{
    const std::optional<DeviceId> d = probe(kind);
    return d ? d->ordinal : -1;
}

int incin_host_detect_device(const int32_t* pref, int32_t n, int32_t* kind, int32_t* ordinal)
{
    const DeviceId d = detect_device_in(n < 0 ? preference() : std::vector<int32_t>(pref, pref + n));
    *kind = d.kind;
    *ordinal = d.ordinal;
    return 0;
}

}  // extern "C"
