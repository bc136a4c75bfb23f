#include "rocm_conformance.hpp"

#include <cmath>
#include <cstring>
#include <exception>
#include <functional>

#include "../../incin_amd/host/rocm_backend.hpp"
#include "../../incin_amd/host/rocm_capability.hpp"
#include "../../incin_amd/host/rocm_exec.hpp"

namespace incin_rocm_host {
namespace conformance {
namespace cap = capability;

bool Tolerance::accepts(double expected, double actual) const
{
    if (expected == actual) return true;
    if (!std::isfinite(expected) || !std::isfinite(actual)) return false;      // non-finite only where the expectation is
    const double diff = std::fabs(expected - actual);
    return diff <= absolute || diff <= relative * std::fabs(expected);
}

bool Report::passed() const { return count(Check::Outcome::Failed) == 0; }
int Report::count(Check::Outcome o) const
{
    int n = 0;
    for (const Check& c : checks) n += c.outcome == o;
    return n;
}
std::string Report::to_text() const
{
    std::string out = "conformance: " + backend + "\n";
    for (const Check& c : checks) {
        if (c.outcome == Check::Outcome::Passed) out += "  pass  " + c.name + "\n";
        else if (c.outcome == Check::Outcome::Skipped) out += "  skip  " + c.name + " (" + c.why + ")\n";
        else out += "  FAIL  " + c.name + ": " + c.why + "\n";
    }
    return out;
}

namespace {
// a check body returns "" on success, else what went wrong; an exception is a failure too (the contract is a
// returned error, never an unwinding one)
Check guarded(const char* name, const std::function<std::string()>& body)
{
    try {
        const std::string why = body();
        return Check{why.empty() ? Check::Outcome::Passed : Check::Outcome::Failed, name, why};
    } catch (const std::exception& e) {
        return Check{Check::Outcome::Failed, name, std::string("threw ") + e.what() + "; the contract requires a returned error"};
    } catch (...) {
        return Check{Check::Outcome::Failed, name, "threw; the contract requires a returned error"};
    }
}

struct Subject {
    int device;
    std::string storage(const std::vector<int64_t>& dims, const std::vector<float>& values, RocmStorage* out) const
    {
        Error e = RocmBackend::from_bytes(values.data(), values.size() * sizeof(float), dims, DType::F32, device, out);
        return e ? e.message : "";
    }
    std::string values(const RocmStorage& s, std::vector<float>* out) const
    {
        std::vector<uint8_t> raw;
        if (Error e = RocmBackend::to_bytes(s, &raw)) return e.message;
        out->resize(raw.size() / sizeof(float));
        if (!raw.empty()) std::memcpy(out->data(), raw.data(), raw.size());
        return "";
    }
};

cap::CapabilityQuery query(cap::OperationKind op, int rank)
{
    return cap::CapabilityQuery{op, cap::DTypeId::F32, cap::LayoutClass::Contiguous, rank, false, cap::MathMode::Precise};
}

std::string dims_str(const std::vector<int64_t>& s)
{
    std::string o = "[";
    for (size_t i = 0; i < s.size(); ++i) o += (i ? ", " : "") + std::to_string(s[i]);
    return o + "]";
}

std::string round_trip(const Subject& s)
{
    const std::vector<float> values = {1.0f, -2.5f, 0.0f, 4.25f, 7.5f, -0.125f};
    RocmStorage st;
    if (std::string e = s.storage({2, 3}, values, &st); !e.empty()) return e;
    std::vector<float> read;
    if (std::string e = s.values(st, &read); !e.empty()) return e;
    if (read.size() != values.size())
        return "wrote " + std::to_string(values.size()) + " values and read back " + std::to_string(read.size());
    for (size_t i = 0; i < values.size(); ++i)
        if (std::memcmp(&values[i], &read[i], sizeof(float)) != 0)
            return "value " + std::to_string(i) + " changed on a round trip: wrote " + std::to_string(values[i]) + ", read " +
                   std::to_string(read[i]);
    return "";
}

std::string metadata_agrees(const Subject& s)
{
    RocmStorage st;
    if (std::string e = s.storage({2, 3}, {1, 2, 3, 4, 5, 6}, &st); !e.empty()) return e;
    if (st.shape != std::vector<int64_t>{2, 3}) return "storage built as [2, 3] reports shape " + dims_str(st.shape);
    if (st.dtype != DType::F32) return "f32 storage reports another dtype; the descriptor path keys on this";
    if (st.numel() != 6) return "shape " + dims_str(st.shape) + " has " + std::to_string(st.numel()) + " elements, not 6";
    if (st.strides.size() != st.shape.size())
        return std::to_string(st.strides.size()) + " strides for a rank-" + std::to_string(st.shape.size()) + " shape";
    return "";
}

std::vector<Check> skipped(const std::vector<const char*>& names, const cap::SupportLevel& support)
{
    std::vector<Check> out;
    for (const char* n : names) out.push_back(Check{Check::Outcome::Skipped, n, support.reason.to_string()});
    return out;
}

// This mirror has no matmul executor; the registry must say so, and then these are skips, not passes.
bool execute_matmul(const Subject&) { return false; }

std::vector<Check> matmul_checks(const Subject& s)
{
    const cap::SupportLevel support = cap::support(cap::DeviceKind::Rocm, query(cap::OperationKind::MatMul, 2));
    const std::vector<const char*> names = {"matmul_is_within_tolerance", "matmul_output_matches_its_descriptor",
                                            "matmul_rejects_a_wrong_input_count"};
    if (!support.is_supported()) return skipped(names, support);
    std::vector<Check> out;
    for (const char* n : names)
        out.push_back(guarded(n, [&] { return execute_matmul(s) ? std::string() : std::string("the registry advertises matmul and no executor exists"); }));
    return out;
}

std::vector<Check> reshape_checks(const Subject& s)
{
    const cap::SupportLevel support = cap::support(cap::DeviceKind::Rocm, query(cap::OperationKind::Reshape, 2));
    if (!support.is_supported()) return skipped({"reshape_preserves_element_order", "reshape_rejects_a_mismatched_operand"}, support);
    const std::vector<float> values = {1, 2, 3, 4, 5, 6};
    return {
        guarded("reshape_preserves_element_order", [&]() -> std::string {
            ReshapeSpec spec;
            if (Error e = lower_reshape({2, 3}, {3, 2}, &spec)) return "the harness could not lower reshape: " + e.message;
            RocmStorage in, o;
            if (std::string e = s.storage({2, 3}, values, &in); !e.empty()) return e;
            if (Error e = execute(spec, {&in}, &o)) return e.message;
            std::vector<float> got;
            if (std::string e = s.values(o, &got); !e.empty()) return e;
            if (got.size() != values.size())
                return "reshape changed the element count from " + std::to_string(values.size()) + " to " + std::to_string(got.size());
            for (size_t i = 0; i < values.size(); ++i)
                if (!EXACT.accepts(values[i], got[i]))
                    return "element " + std::to_string(i) + " is " + std::to_string(got[i]) + " after a reshape of " +
                           std::to_string(values[i]) + "; reshape re-addresses bytes and must not compute";
            return "";
        }),
        guarded("reshape_rejects_a_mismatched_operand", [&]() -> std::string {
            ReshapeSpec spec;
            if (Error e = lower_reshape({2, 3}, {3, 2}, &spec)) return "the harness could not lower reshape: " + e.message;
            RocmStorage wrong, o;
            if (std::string e = s.storage({3, 2}, values, &wrong); !e.empty()) return e;
            if (!execute(spec, {&wrong}, &o))
                return "an operand whose shape disagrees with the validated descriptor was accepted; the executor is the only place that can notice";
            return "";
        }),
    };
}

// Two heads of the hand-composed case the reference's tensor-parallel tests check against a closed form
// (crates/incin/tests/tp2_network.rs:339-366): S = 2, D = 1, scale 1, no mask.  The expectation is evaluated here in
// f64 from the definition, not taken from the backend under test.
void closed_form(const float q[2], const float k[2], const float v[2], double out[2])
{
    for (int i = 0; i < 2; ++i) {
        const double s0 = (double)q[i] * k[0], s1 = (double)q[i] * k[1], m = std::fmax(s0, s1);
        const double e0 = std::exp(s0 - m), e1 = std::exp(s1 - m);
        out[i] = (e0 * v[0] + e1 * v[1]) / (e0 + e1);
    }
}

std::vector<Check> attention_checks(const Subject& s)
{
    const cap::SupportLevel support = cap::support(cap::DeviceKind::Rocm, query(cap::OperationKind::Attention, 3));
    const std::vector<const char*> names = {"attention_is_within_tolerance", "attention_output_matches_its_descriptor",
                                            "attention_rejects_a_wrong_input_count", "attention_descriptor_facts_equal_an_explicit_mask"};
    if (!support.is_supported()) return skipped(names, support);
    const std::vector<float> q = {1, 2, 0.5f, -0.5f}, k = {1, -1, 2, 1}, v = {3, 5, 7, 11};      // [2 heads, 2, 1]
    auto lower = [](AttentionSpec* spec, bool causal) {
        return lower_attention({2, 2, 1}, {2, 2, 1}, {2, 2, 1}, DType::F32, causal, std::nullopt, 1.0, spec);
    };
    return {
        guarded(names[0], [&]() -> std::string {
            AttentionSpec spec;
            if (Error e = lower(&spec, false)) return "the harness could not lower attention: " + e.message;
            RocmStorage sq, sk, sv, o;
            for (auto [st, vals] : {std::pair{&sq, &q}, std::pair{&sk, &k}, std::pair{&sv, &v}})
                if (std::string e = s.storage({2, 2, 1}, *vals, st); !e.empty()) return e;
            if (Error e = execute(spec, {&sq, &sk, &sv}, &o)) return e.message;
            std::vector<float> got;
            if (std::string e = s.values(o, &got); !e.empty()) return e;
            if (got.size() != 4) return "two heads of two queries produced " + std::to_string(got.size()) + " values, not 4";
            for (int h = 0; h < 2; ++h) {
                double want[2];
                closed_form(&q[2 * h], &k[2 * h], &v[2 * h], want);
                for (int i = 0; i < 2; ++i)
                    if (!F32_ACCUMULATED.accepts(want[i], got[2 * h + i]))
                        return "head " + std::to_string(h) + " query " + std::to_string(i) + " is " + std::to_string(got[2 * h + i]) +
                               ", outside 1e-5 of " + std::to_string(want[i]);
            }
            return "";
        }),
        guarded(names[1], [&]() -> std::string {
            AttentionSpec spec;
            // grouped queries over a longer key sequence: q [2, 3, 5, 8] against k, v [2, 1, 7, 8] / [2, 1, 7, 4]
            if (Error e = lower_attention({2, 3, 5, 8}, {2, 1, 7, 8}, {2, 1, 7, 4}, DType::F32, true, std::nullopt, std::nullopt, &spec))
                return "the harness could not lower attention: " + e.message;
            if (spec.out_dims != std::vector<int64_t>{2, 3, 5, 4}) return "the rule proves " + dims_str(spec.out_dims) + " for the output, not [2, 3, 5, 4]";
            RocmStorage sq, sk, sv, o;
            if (std::string e = s.storage({2, 3, 5, 8}, std::vector<float>(240, 0.25f), &sq); !e.empty()) return e;
            if (std::string e = s.storage({2, 1, 7, 8}, std::vector<float>(112, 0.5f), &sk); !e.empty()) return e;
            if (std::string e = s.storage({2, 1, 7, 4}, std::vector<float>(56, 2.0f), &sv); !e.empty()) return e;
            if (Error e = execute(spec, {&sq, &sk, &sv}, &o)) return e.message;
            if (o.shape != spec.out_dims)
                return "the validated descriptor says " + dims_str(spec.out_dims) + " and the output reports " + dims_str(o.shape);
            if (o.dtype != DType::F32) return "f32 operands produced another dtype";
            std::vector<float> got;
            if (std::string e = s.values(o, &got); !e.empty()) return e;
            for (float x : got)
                if (!F32_ACCUMULATED.accepts(2.0, x)) return "a weighted mean of values that are all 2 came out as " + std::to_string(x);
            return "";
        }),
        guarded(names[2], [&]() -> std::string {
            AttentionSpec spec;
            if (Error e = lower(&spec, false)) return "the harness could not lower attention: " + e.message;
            RocmStorage sq, sk, o;
            if (std::string e = s.storage({2, 2, 1}, q, &sq); !e.empty()) return e;
            if (std::string e = s.storage({2, 2, 1}, k, &sk); !e.empty()) return e;
            if (!execute(spec, {&sq, &sk}, &o)) return "two operands were accepted for a three-operand attention; arity is the executor's to check";
            RocmStorage wrong;
            if (std::string e = s.storage({2, 1, 2}, q, &wrong); !e.empty()) return e;
            if (!execute(spec, {&wrong, &sk, &sk}, &o)) return "an operand whose shape disagrees with the validated descriptor was accepted";
            return "";
        }),
        guarded(names[3], [&]() -> std::string {
            // causal alignment stated by the descriptor = the operator given the explicit additive mask
            AttentionSpec spec;
            if (Error e = lower(&spec, true)) return "the harness could not lower attention: " + e.message;
            RocmStorage sq, sk, sv, sm, a, b;
            for (auto [st, vals] : {std::pair{&sq, &q}, std::pair{&sk, &k}, std::pair{&sv, &v}})
                if (std::string e = s.storage({2, 2, 1}, *vals, st); !e.empty()) return e;
            const float ninf = -INFINITY;
            if (std::string e = s.storage({2, 2}, {0.0f, ninf, 0.0f, 0.0f}, &sm); !e.empty()) return e;
            if (Error e = execute(spec, {&sq, &sk, &sv}, &a)) return e.message;
            if (Error e = RocmBackend::scaled_dot_product_attention(sq, sk, sv, &sm, 1.0, &b)) return e.message;
            std::vector<float> ga, gb;
            if (std::string e = s.values(a, &ga); !e.empty()) return e;
            if (std::string e = s.values(b, &gb); !e.empty()) return e;
            for (size_t i = 0; i < ga.size(); ++i)
                if (!F32_ACCUMULATED.accepts(gb[i], ga[i]))
                    return "element " + std::to_string(i) + ": " + std::to_string(ga[i]) + " from the descriptor's causal flag, " +
                           std::to_string(gb[i]) + " from the explicit mask";
            return "";
        }),
    };
}

// Gradients of the same hand-composed heads for an upstream gradient g, evaluated in f64 from the definition (the chain
// the reference's tape walks, cpu/tape.rs:149-176): P = softmax rows, dV_j = sum_i P_ij g_i, dP_ij = g_i v_j,
// dS_ij = P_ij (dP_ij - sum_l P_il dP_il), dq_i = sum_j dS_ij k_j, dk_j = sum_i dS_ij q_i (scale 1, D = 1).
void closed_form_gradients(const float q[2], const float k[2], const float v[2], const float g[2], double dq[2], double dk[2], double dv[2])
{
    double P[2][2], dS[2][2];
    for (int i = 0; i < 2; ++i) {
        const double s0 = (double)q[i] * k[0], s1 = (double)q[i] * k[1], m = std::fmax(s0, s1);
        const double e0 = std::exp(s0 - m), e1 = std::exp(s1 - m);
        P[i][0] = e0 / (e0 + e1);
        P[i][1] = e1 / (e0 + e1);
        const double dP0 = (double)g[i] * v[0], dP1 = (double)g[i] * v[1], D = P[i][0] * dP0 + P[i][1] * dP1;
        dS[i][0] = P[i][0] * (dP0 - D);
        dS[i][1] = P[i][1] * (dP1 - D);
        dq[i] = dS[i][0] * k[0] + dS[i][1] * k[1];
    }
    for (int j = 0; j < 2; ++j) {
        dv[j] = P[0][j] * g[0] + P[1][j] * g[1];
        dk[j] = dS[0][j] * q[0] + dS[1][j] * q[1];
    }
}

std::vector<Check> attention_training_checks(const Subject& s)
{
    cap::CapabilityQuery tq = query(cap::OperationKind::Attention, 3);
    tq.training = true;
    const cap::SupportLevel support = cap::support(cap::DeviceKind::Rocm, tq);
    const std::vector<const char*> names = {"attention_gradients_are_within_tolerance", "attention_gradients_have_their_operands_shapes"};
    if (!support.is_supported()) return skipped(names, support);
    const std::vector<float> q = {1, 2, 0.5f, -0.5f}, k = {1, -1, 2, 1}, v = {3, 5, 7, 11}, g = {1, -2, 0.5f, 3};      // [2 heads, 2, 1]
    return {
        guarded(names[0], [&]() -> std::string {
            RocmStorage sq, sk, sv, sg, o;
            for (auto [st, vals] : {std::pair{&sq, &q}, std::pair{&sk, &k}, std::pair{&sv, &v}, std::pair{&sg, &g}})
                if (std::string e = s.storage({2, 2, 1}, *vals, st); !e.empty()) return e;
            RocmBackend::AttentionGrads grads;
            if (Error e = RocmBackend::attention_backward(sq, sk, sv, nullptr, 1.0, RocmBackend::MaskFacts{}, sg, &o, &grads)) return e.message;
            std::vector<float> gq, gk, gv;
            if (std::string e = s.values(grads.dq, &gq); !e.empty()) return e;
            if (std::string e = s.values(grads.dk, &gk); !e.empty()) return e;
            if (std::string e = s.values(grads.dv, &gv); !e.empty()) return e;
            if (gq.size() != 4 || gk.size() != 4 || gv.size() != 4) return "gradients of [2, 2, 1] operands do not hold 4 values each";
            for (int h = 0; h < 2; ++h) {
                double wq[2], wk[2], wv[2];
                closed_form_gradients(&q[2 * h], &k[2 * h], &v[2 * h], &g[2 * h], wq, wk, wv);
                for (int i = 0; i < 2; ++i) {
                    const std::pair<const char*, std::pair<double, float>> rows[] = {
                        {"dq", {wq[i], gq[2 * h + i]}}, {"dk", {wk[i], gk[2 * h + i]}}, {"dv", {wv[i], gv[2 * h + i]}}};
                    for (const auto& [what, pr] : rows)
                        if (!F32_ACCUMULATED.accepts(pr.first, pr.second))
                            return std::string(what) + " of head " + std::to_string(h) + " row " + std::to_string(i) + " is " +
                                   std::to_string(pr.second) + ", outside 1e-5 of " + std::to_string(pr.first);
                }
            }
            return "";
        }),
        guarded(names[1], [&]() -> std::string {
            // grouped queries: k and v shared by 3 query heads get gradients of their own shape, summed over the group; with
            // all values equal the output does not depend on the weights, so dq = dk = 0 and every dv row adds up the upstream rows
            RocmStorage sq, sk, sv, sg, o;
            if (std::string e = s.storage({2, 1, 3, 5, 8}, std::vector<float>(240, 0.25f), &sq); !e.empty()) return e;
            if (std::string e = s.storage({2, 1, 1, 7, 8}, std::vector<float>(112, 0.5f), &sk); !e.empty()) return e;
            if (std::string e = s.storage({2, 1, 1, 7, 4}, std::vector<float>(56, 2.0f), &sv); !e.empty()) return e;
            if (std::string e = s.storage({2, 1, 3, 5, 4}, std::vector<float>(120, 1.0f), &sg); !e.empty()) return e;
            RocmBackend::AttentionGrads grads;
            if (Error e = RocmBackend::attention_backward(sq, sk, sv, nullptr, std::nullopt, RocmBackend::MaskFacts{}, sg, &o, &grads)) return e.message;
            if (grads.dq.shape != sq.shape || grads.dk.shape != sk.shape || grads.dv.shape != sv.shape)
                return "gradients report " + dims_str(grads.dq.shape) + ", " + dims_str(grads.dk.shape) + ", " + dims_str(grads.dv.shape) +
                       " for operands " + dims_str(sq.shape) + ", " + dims_str(sk.shape) + ", " + dims_str(sv.shape);
            std::vector<float> gq, gk, gv;
            if (std::string e = s.values(grads.dq, &gq); !e.empty()) return e;
            if (std::string e = s.values(grads.dk, &gk); !e.empty()) return e;
            if (std::string e = s.values(grads.dv, &gv); !e.empty()) return e;
            for (float x : gq)
                if (!F32_ACCUMULATED.accepts(0.0, x)) return "dq of an output that does not depend on q came out as " + std::to_string(x);
            for (float x : gk)
                if (!F32_ACCUMULATED.accepts(0.0, x)) return "dk of an output that does not depend on k came out as " + std::to_string(x);
            // uniform weights 1/7 from 3 heads x 5 rows of ones: 15 / 7 per element
            for (float x : gv)
                if (!F32_ACCUMULATED.accepts(15.0 / 7.0, x)) return "dv under uniform weights came out as " + std::to_string(x) + ", not 15/7";
            return "";
        }),
    };
}

// The runtime-dispatch arm (dispatch.rs:1196-1225): operands held by the rocm backend reach its operator and come back
// wrapped; an operand or a mask held by no backend is an error with the reference's message, not a silent copy.
std::string dispatch_routes(const Subject& s)
{
    const std::vector<float> q = {1, 2, 0.5f, -0.5f}, k = {1, -1, 2, 1}, v = {3, 5, 7, 11};
    RocmStorage sq, sk, sv;
    for (auto [st, vals] : {std::pair{&sq, &q}, std::pair{&sk, &k}, std::pair{&sv, &v}})
        if (std::string e = s.storage({2, 2, 1}, *vals, st); !e.empty()) return e;
    const DispatchStorage dq = DispatchStorage::on_rocm(sq), dk = DispatchStorage::on_rocm(sk), dv = DispatchStorage::on_rocm(sv), nowhere;
    DispatchStorage out;
    if (Error e = DispatchBackend::scaled_dot_product_attention(dq, dk, dv, nullptr, 1.0, &out)) return e.message;
    if (out.holder != DispatchStorage::Holder::Rocm) return "the result of a rocm attention is not held by rocm";
    std::vector<float> got;
    if (std::string e = s.values(out.rocm, &got); !e.empty()) return e;
    for (int h = 0; h < 2; ++h) {
        double want[2];
        closed_form(&q[2 * h], &k[2 * h], &v[2 * h], want);
        for (int i = 0; i < 2; ++i)
            if (!F32_ACCUMULATED.accepts(want[i], got[2 * h + i])) return "dispatched attention is outside 1e-5 of the closed form";
    }
    Error e = DispatchBackend::scaled_dot_product_attention(dq, nowhere, dv, nullptr, 1.0, &out);
    if (!e || e.message != "mismatched backends in SDPA") return "an operand held by no backend gave: " + (e ? e.message : std::string("success"));
    e = DispatchBackend::scaled_dot_product_attention(dq, dk, dv, &nowhere, 1.0, &out);
    if (!e || e.message != "mismatched mask backend") return "a mask held by no backend gave: " + (e ? e.message : std::string("success"));
    return "";
}

std::string registry_agrees(const Subject& s)
{
    auto word = [](bool b, const char* yes, const char* no) { return std::string(b ? yes : no); };
    const bool matmul_claimed = cap::support(cap::DeviceKind::Rocm, query(cap::OperationKind::MatMul, 2)).is_supported();
    const bool matmul_ran = execute_matmul(s);
    if (matmul_claimed != matmul_ran)
        return "the registry says matmul is " + word(matmul_claimed, "supported", "unsupported") + " and executing it " +
               word(matmul_ran, "succeeded", "failed");
    const std::vector<float> values = {1, 2, 3, 4, 5, 6};
    const bool reshape_claimed = cap::support(cap::DeviceKind::Rocm, query(cap::OperationKind::Reshape, 2)).is_supported();
    ReshapeSpec rs;
    if (Error e = lower_reshape({2, 3}, {3, 2}, &rs)) return "the harness could not lower reshape: " + e.message;
    RocmStorage in, o;
    if (std::string e = s.storage({2, 3}, values, &in); !e.empty()) return e;
    const bool reshape_ran = !execute(rs, {&in}, &o);
    if (reshape_claimed != reshape_ran)
        return "the registry says reshape is " + word(reshape_claimed, "supported", "unsupported") + " and executing it " +
               word(reshape_ran, "succeeded", "failed");
    const bool attn_claimed = cap::support(cap::DeviceKind::Rocm, query(cap::OperationKind::Attention, 2)).is_supported();
    AttentionSpec as;
    if (Error e = lower_attention({2, 3}, {2, 3}, {2, 3}, DType::F32, false, std::nullopt, std::nullopt, &as))
        return "the harness could not lower attention: " + e.message;
    const bool attn_ran = !execute(as, {&in, &in, &in}, &o);
    if (attn_claimed != attn_ran)
        return "the registry says attention is " + word(attn_claimed, "supported", "unsupported") + " and executing it " +
               word(attn_ran, "succeeded", "failed");
    cap::CapabilityQuery training = query(cap::OperationKind::Attention, 2);
    training.training = true;
    const bool train_claimed = cap::support(cap::DeviceKind::Rocm, training).is_supported();
    RocmBackend::AttentionGrads grads;
    const bool train_ran = !RocmBackend::attention_backward(in, in, in, nullptr, std::nullopt, RocmBackend::MaskFacts{}, in, &o, &grads);
    if (train_claimed != train_ran)
        return "the registry says training attention is " + word(train_claimed, "supported", "unsupported") + " and its backward " +
               word(train_ran, "succeeded", "failed");
    // a dtype the storage cannot represent must be refused by the registry rather than discovered in a kernel
    bool refuses = false;
    for (cap::DTypeId d : {cap::DTypeId::Q8_0, cap::DTypeId::F64, cap::DTypeId::U8}) {
        cap::CapabilityQuery probe = query(cap::OperationKind::Attention, 2);
        probe.dtype = d;
        refuses = refuses || !cap::support(cap::DeviceKind::Rocm, probe).is_supported();
    }
    if (!refuses) return "the registry claims attention for every dtype probed, including Q8_0; a registry that never says no cannot be planned against";
    // and a view the registry refuses (last axis not dense) must be refused by the executor
    cap::CapabilityQuery strided = query(cap::OperationKind::Attention, 2);
    strided.layout = cap::LayoutClass::Strided;
    RocmStorage t;
    if (Error e = RocmBackend::transpose(in, 0, 1, &t)) return e.message;
    AttentionSpec ts;
    if (Error e = lower_attention({3, 2}, {3, 2}, {3, 2}, DType::F32, false, std::nullopt, std::nullopt, &ts))
        return "the harness could not lower attention: " + e.message;
    const bool strided_ran = !execute(ts, {&t, &t, &t}, &o);
    if (cap::support(cap::DeviceKind::Rocm, strided).is_supported() != strided_ran)
        return "the registry and the executor disagree about a view whose last axis is not dense";
    return "";
}
}  // namespace

Report run(int device)
{
    const Subject s{device};
    Report r;
    r.backend = "rocm:" + std::to_string(device);
    r.checks.push_back(guarded("storage_round_trips_its_values", [&] { return round_trip(s); }));
    r.checks.push_back(guarded("metadata_describes_the_tensor_it_came_from", [&] { return metadata_agrees(s); }));
    for (Check& c : matmul_checks(s)) r.checks.push_back(std::move(c));
    for (Check& c : reshape_checks(s)) r.checks.push_back(std::move(c));
    for (Check& c : attention_checks(s)) r.checks.push_back(std::move(c));
    for (Check& c : attention_training_checks(s)) r.checks.push_back(std::move(c));
    r.checks.push_back(guarded("dispatch_routes_attention_to_the_holder_of_its_operands", [&] { return dispatch_routes(s); }));
    r.checks.push_back(guarded("the_registry_and_the_executor_agree", [&] { return registry_agrees(s); }));
    return r;
}

}  // namespace conformance
}  // namespace incin_rocm_host

// Flat C entry for the Python test: the report text (at most capacity - 1 bytes written, full length returned) and how
// many checks passed, were skipped, failed.
extern "C" size_t incin_conformance_run(int32_t device, char* text, size_t capacity, int32_t* passed, int32_t* skipped, int32_t* failed)
{
    namespace conf = incin_rocm_host::conformance;
    const conf::Report r = conf::run(device);
    if (passed) *passed = r.count(conf::Check::Outcome::Passed);
    if (skipped) *skipped = r.count(conf::Check::Outcome::Skipped);
    if (failed) *failed = r.count(conf::Check::Outcome::Failed);
    const std::string t = r.to_text();
    if (text && capacity) {
        const size_t n = t.size() < capacity - 1 ? t.size() : capacity - 1;
        std::memcpy(text, t.data(), n);
        text[n] = 0;
    }
    return t.size();
}
