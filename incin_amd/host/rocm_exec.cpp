#include "rocm_exec.hpp"

#include <string>

#include "../../include/incin_rocm.h"

namespace incin_rocm_host {
namespace {
Error ok() { return Error{}; }
Error bad(const std::string& m) { return Error{ErrorKind::ShapeMismatch, m}; }
std::string dims_str(const std::vector<int64_t>& s)
{
    std::string o = "[";
    for (size_t i = 0; i < s.size(); ++i) o += (i ? ", " : "") + std::to_string(s[i]);
    return o + "]";
}
const char* OP = "scaled_dot_product_attention";
}  // namespace

Error lower_attention(const std::vector<int64_t>& q, const std::vector<int64_t>& k, const std::vector<int64_t>& v, DType dtype,
                      bool causal, const std::optional<std::vector<int32_t>>& kv_lens, std::optional<double> scale,
                      AttentionSpec* out, const std::optional<std::vector<int32_t>>& q_lens)
{
    if (q.size() < 2 || k.size() < 2 || v.size() < 2)
        return bad(std::string(OP) + ": operands need rank >= 2; got q " + dims_str(q) + ", k " + dims_str(k) + ", v " + dims_str(v));
    for (const auto* s : {&q, &k, &v})
        for (int64_t d : *s)
            if (d < 0) return bad(std::string(OP) + ": negative extent in " + dims_str(*s));
    const int64_t Sq = q[q.size() - 2], D = q.back(), Skv = k[k.size() - 2], Dv = v.back();
    if (k.back() != D) return bad(std::string(OP) + ": q and k inner dims must match: q " + dims_str(q) + ", k " + dims_str(k));
    if (v[v.size() - 2] != Skv) return bad(std::string(OP) + ": k and v key counts must match: k " + dims_str(k) + ", v " + dims_str(v));
    // batch axes: broadcast(broadcast(q, k), v)
    const std::vector<int64_t> qb(q.begin(), q.end() - 2), kb(k.begin(), k.end() - 2), vb(v.begin(), v.end() - 2);
    std::vector<int64_t> t, b;
    if (Error e = broadcast_shape(qb, kb, &t)) return bad(std::string(OP) + ": " + e.message);
    if (Error e = broadcast_shape(t, vb, &b)) return bad(std::string(OP) + ": " + e.message);
    AttentionSpec s;
    s.q_dims = q; s.k_dims = k; s.v_dims = v;
    s.out_dims = b;
    s.out_dims.push_back(Sq);
    s.out_dims.push_back(Dv);
    // grouped queries: the last batch axis is > 1 for q and 1 for k and v
    if (!b.empty() && qb.size() == b.size() && kb.size() == b.size() && vb.size() == b.size() && qb.back() > 1 && kb.back() == 1 &&
        vb.back() == 1 && b.size() >= 2)
        s.group = qb.back();
    for (int which = 0; which < 2; ++which) {
        const std::optional<std::vector<int32_t>>& lens = which ? q_lens : kv_lens;
        const int64_t limit = which ? Sq : Skv;
        const char* what = which ? "query" : "key";
        if (!lens) continue;
        // one count per index of the batch axis: none below rank 4 (one set of sequences), the first axis at rank 4, the
        // axis before [kv heads] or [kv heads, group] above
        const int nb = (int)b.size();
        const int b_ax = nb <= 1 ? -1 : nb == 2 ? 0 : (s.group > 1 ? nb - 3 : nb - 2);      // a single batch axis counts heads
        const int64_t B = b_ax >= 0 ? b[b_ax] : 1;
        if ((int64_t)lens->size() != B)
            return bad(std::string(OP) + ": " + std::to_string(lens->size()) + " " + what + " counts for a batch axis of " + std::to_string(B));
        for (int32_t n : *lens)
            if (n < 0 || n > limit) return bad(std::string(OP) + ": " + what + " count " + std::to_string(n) + " outside 0..=" + std::to_string(limit));
    }
    if (scale && !(*scale == *scale)) return Error{ErrorKind::Msg, std::string(OP) + ": scale is NaN"};
    s.causal = causal;
    s.kv_lens = kv_lens;
    s.q_lens = q_lens;
    s.scale = scale;
    s.dtype = dtype;
    *out = std::move(s);
    return ok();
}

Error lower_reshape(const std::vector<int64_t>& in, const std::vector<int64_t>& outd, ReshapeSpec* out)
{
    int64_t a = 1, b = 1;
    for (int64_t d : in) a *= d;
    for (int64_t d : outd) b *= d;
    for (const auto* s : {&in, &outd})
        for (int64_t d : *s)
            if (d < 0) return bad("reshape: negative extent in " + dims_str(*s));
    if (a != b) return bad("reshape: " + dims_str(in) + " has " + std::to_string(a) + " elements, " + dims_str(outd) + " has " + std::to_string(b));
    *out = ReshapeSpec{in, outd};
    return ok();
}

Error execute(const AttentionSpec& spec, const std::vector<const RocmStorage*>& inputs, RocmStorage* out)
{
    if (inputs.size() != 3)
        return bad(std::string(OP) + ": the descriptor takes 3 operands (q, k, v), " + std::to_string(inputs.size()) + " given");
    const RocmStorage &q = *inputs[0], &k = *inputs[1], &v = *inputs[2];
    if (q.shape != spec.q_dims || k.shape != spec.k_dims || v.shape != spec.v_dims)
        return bad(std::string(OP) + ": operands q " + dims_str(q.shape) + ", k " + dims_str(k.shape) + ", v " + dims_str(v.shape) +
                   " disagree with the validated descriptor q " + dims_str(spec.q_dims) + ", k " + dims_str(spec.k_dims) + ", v " +
                   dims_str(spec.v_dims));
    if (q.dtype != spec.dtype || k.dtype != spec.dtype || v.dtype != spec.dtype)
        return Error{ErrorKind::DTypeStorageMismatch, std::string(OP) + ": operand dtypes disagree with the validated descriptor"};
    RocmBackend::MaskFacts facts;
    facts.causal = spec.causal;
    if (spec.kv_lens) {
        if (Error e = RocmBackend::upload_i32(*spec.kv_lens, q.device, &facts.kv_lens)) return e;
        facts.kv_lens_count = (int64_t)spec.kv_lens->size();
    }
    if (spec.q_lens) {
        if (Error e = RocmBackend::upload_i32(*spec.q_lens, q.device, &facts.q_lens)) return e;
        facts.q_lens_count = (int64_t)spec.q_lens->size();
    }
    RocmStorage o;
    if (Error e = RocmBackend::attention(q, k, v, nullptr, spec.scale, facts, &o)) return e;
    if (o.shape != spec.out_dims)
        return Error{ErrorKind::Msg, std::string(OP) + ": produced " + dims_str(o.shape) + ", the descriptor proves " + dims_str(spec.out_dims)};
    // (the key counts are still being read by the launch: their buffers are released in stream order)
    *out = std::move(o);
    return ok();
}

Error execute(const ReshapeSpec& spec, const std::vector<const RocmStorage*>& inputs, RocmStorage* out)
{
    if (inputs.size() != 1) return bad("reshape: the descriptor takes 1 operand, " + std::to_string(inputs.size()) + " given");
    if (inputs[0]->shape != spec.in_dims)
        return bad("reshape: operand " + dims_str(inputs[0]->shape) + " disagrees with the validated descriptor " + dims_str(spec.in_dims));
    return RocmBackend::reshape(*inputs[0], spec.out_dims, out);
}

// ---- detection ------------------------------------------------------------------------------------------------
bool is_compiled_in(int32_t kind) { return kind == 4; }

std::optional<DeviceId> probe(int32_t kind)
{
    if (kind != 4) return std::nullopt;
    int n = 0;
    if (incin_rocm_device_count(&n) != 0 || n <= 0) return std::nullopt;
    // a listed device can still be unusable (no permission, exhausted): only doing what comes next proves it can be done
    void* p = nullptr;
    if (incin_rocm_alloc(0, 256, &p) != 0) return std::nullopt;
    incin_rocm_free(0, p);
    return DeviceId{4, 0};
}

const std::vector<int32_t>& preference()
{
    static const std::vector<int32_t> order = {1, 4, 3, 2, 0};
    return order;
}

DeviceId detect_device_in(const std::vector<int32_t>& pref)
{
    for (int32_t kind : pref)
        if (auto d = probe(kind)) return *d;
    return DeviceId{0, 0};
}

DispatchStorage DispatchStorage::on_rocm(RocmStorage s)
{
    DispatchStorage d;
    d.holder = Holder::Rocm;
    d.rocm = std::move(s);
    return d;
}

Error DispatchBackend::scaled_dot_product_attention(const DispatchStorage& q, const DispatchStorage& k, const DispatchStorage& v,
                                                    const DispatchStorage* mask, std::optional<double> scale, DispatchStorage* out)
{
    using H = DispatchStorage::Holder;
    if (q.holder == H::Rocm && k.holder == H::Rocm && v.holder == H::Rocm) {
        if (mask && mask->holder != H::Rocm) return Error{ErrorKind::Msg, "mismatched mask backend"};
        RocmStorage o;
        if (Error e = RocmBackend::scaled_dot_product_attention(q.rocm, k.rocm, v.rocm, mask ? &mask->rocm : nullptr, scale, &o)) return e;
        *out = DispatchStorage::on_rocm(std::move(o));
        return Error{};
    }
    return Error{ErrorKind::Msg, "mismatched backends in SDPA"};
}

}  // namespace incin_rocm_host
