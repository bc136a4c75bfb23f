// Test-side harness (built into tests/native/libincin_rocm_conformance.so, not into the product libraries): the backend
// conformance suite for the rocm backend mirror: the checks of
// crates/incin-backends/src/external/conformance.rs:199-216 (storage round trip, metadata, matmul and reshape through
// validated descriptors, registry and executor agreeing), reported the same way (pass / skip with the registry's
// reason / FAIL with what went wrong, :93-160), plus the same three kinds of check for attention.  An operation the
// registry does not advertise is skipped with the registry's refusal as the reason, never silently passed.
#pragma once
#include <string>
#include <vector>

namespace incin_rocm_host {
namespace conformance {

struct Tolerance {
    double absolute, relative;
    bool accepts(double expected, double actual) const;
};
constexpr Tolerance EXACT{0.0, 0.0};
constexpr Tolerance F32_ACCUMULATED{1e-5, 1e-5};      // external/conformance.rs:73-77

struct Check {
    enum class Outcome { Passed, Skipped, Failed } outcome;
    std::string name, why;
};

struct Report {
    std::string backend;
    std::vector<Check> checks;
    bool passed() const;
    int count(Check::Outcome o) const;
    std::string to_text() const;
};

// Runs every check against device `device` of the rocm backend.
Report run(int device);

}  // namespace conformance
}  // namespace incin_rocm_host
