"""The capability registry of the rocm backend (C++ host mirror), tested the way the reference tests its
own tables (crates/incin-backends/tests/capability_matrix.rs:32-86 boundary cases of every registration,
:88-220 refusals carry the documented constraint; tests/generated_docs.rs: the checked-in table is what the
renderer produces).  Nothing here touches a device."""
import os

import pytest

from incin_amd import rocm_capability as RC

Q = RC.CapabilityQuery
HERE = os.path.dirname(os.path.abspath(__file__))
DOC = os.path.join(os.path.dirname(HERE), "incin_amd", "host", "capabilities_rocm.md")


def test_enumerations_spell_like_the_reference():
    # incin-core/src/shapes/error.rs:140-165, exec/meta.rs:41-51, exec/policy.rs:28-32
    ops = RC.operations()
    assert ops[:8] == ["storage", "fill", "random", "pointwise", "reduction", "normalization", "broadcast", "reshape"]
    assert ops[16] == "matmul" and ops[21] == "adaptive_avg_pool2d" and ops[-1] == "attention"
    assert RC.dtypes() == ["u8", "u32", "i64", "bf16", "f16", "f32", "f64", "q8_0"]
    assert RC.layouts() == ["strided", "contiguous", "scalar-left", "scalar-right", "contiguous-last-axis", "row-wise",
                            "channel-wise"]
    assert RC.math_modes() == ["precise", "fast"]
    assert RC.implementations() == ["native", "composed", "fallback"]
    assert RC.devices() == ["cpu", "cuda", "wgpu", "metal", "rocm"]
    assert RC.max_rank() == 8


@pytest.mark.parametrize("device", ["rocm", "cpu"])
def test_every_registration_generates_supported_boundary_cases_without_fallback(device):
    rules = RC.registrations(device)
    assert rules
    for rule in rules:
        assert rule.dtypes and rule.layouts and rule.math_modes
        assert rule.min_rank <= rule.max_rank
        assert rule.implementation != "fallback"
        for dtype in rule.dtypes:
            for layout in rule.layouts:
                for mode in rule.math_modes:
                    for rank in (rule.min_rank, rule.max_rank):
                        case = Q(rule.operation, dtype, layout, rank, False, mode)
                        assert RC.support(device, case).level == rule.implementation, (device, case)
                        if rule.training:
                            assert RC.support(device, case._replace(training=True)).level == rule.implementation


def test_unsupported_cells_return_the_documented_constraint():
    s = RC.support("rocm", Q("attention", "f64", "contiguous", 4))
    assert (s.level, s.reason, s.message) == ("unsupported", "DType", "dtype F64 is unsupported for attention")
    s = RC.support("rocm", Q("attention", "q8_0", "contiguous", 4))
    assert s.reason == "DType" and s.message == "dtype Q8_0 is unsupported for attention"
    # a view whose last axis is not dense runs through a dense temporary: composed, not native
    assert RC.support("rocm", Q("attention", "bf16", "strided", 4)).level == "composed"
    s = RC.support("rocm", Q("attention", "bf16", "channel-wise", 4))
    assert (s.reason, s.message) == ("Layout", "layout channel-wise is unsupported for attention")
    s = RC.support("rocm", Q("attention", "f32", "contiguous", 1))
    assert (s.reason, s.message) == ("Rank", "rank 1 is unsupported for attention; expected 2..=8")
    assert RC.support("rocm", Q("attention", "bf16", "contiguous", 4, training=True)).level == "native"
    s = RC.support("rocm", Q("reshape", "bf16", "contiguous", 4, training=True))
    assert (s.reason, s.message) == ("Training", "training is unsupported for reshape")
    s = RC.support("rocm", Q("attention", "bf16", "contiguous", 4, math_mode="fast"))
    assert (s.reason, s.message) == ("MathMode", "math mode fast is unsupported for attention")
    # not registered at all: pointwise has no family rule either
    s = RC.support("rocm", Q("pointwise", "f32", "contiguous", 2))
    assert (s.reason, s.message) == ("Operation", "operation pointwise is not registered")
    # matmul resolves through its family (reduction), which this backend does not register
    assert RC.support("rocm", Q("matmul", "f32", "contiguous", 2)).reason == "Operation"
    # the CPU row is trainable but f32 only
    assert RC.support("cpu", Q("attention", "f32", "strided", 8, training=True)).level == "composed"
    assert RC.support("cpu", Q("attention", "bf16", "contiguous", 4)).reason == "DType"


def test_operations_without_rules_of_their_own_resolve_through_their_family():
    # transpose / narrow (slice) and the like are metadata operations: family `storage`
    # (incin-core/src/shapes/error.rs:112-124), answered by the storage rule
    for op in ("transpose", "slice", "permute", "squeeze"):
        assert RC.support("rocm", Q(op, "bf16", "strided", 5)).level == "native"
        assert RC.support("rocm", Q(op, "i64", "contiguous", 5)).reason == "DType"
    # broadcast and reshape have rules of their own, which then are the only ones consulted: reshape re-addresses
    # contiguous storage and gathers any other view into a dense copy first
    assert RC.support("rocm", Q("broadcast", "f16", "row-wise", 8)).level == "native"
    assert RC.support("rocm", Q("reshape", "f16", "contiguous", 8)).level == "native"
    assert RC.support("rocm", Q("reshape", "f16", "strided", 3)).level == "composed"
    s = RC.support("rocm", Q("reshape", "f16", "scalar-left", 3))
    assert (s.reason, s.message) == ("Layout", "layout scalar-left is unsupported for reshape")


@pytest.mark.parametrize("device", ["cuda", "wgpu", "metal"])
def test_other_devices_have_no_registrations_here(device):
    assert RC.registrations(device) == []
    assert RC.support(device, Q("attention", "f32", "contiguous", 4)).reason == "Operation"


def test_checked_in_table_is_what_the_renderer_produces():
    text = RC.docs()
    if os.environ.get("INCIN_DOCS") == "overwrite":
        with open(DOC, "w") as f:
            f.write(text)
    assert open(DOC).read() == text, "regenerate with INCIN_DOCS=overwrite python -m pytest tests/test_capability_registry.py"
    assert "| `attention` | `f32` | `bf16`, `f16`, `f32` |" in text
    assert "| `attention` | `bf16`, `f16`, `f32` | `contiguous`, `row-wise` | 2+ | yes | native |" in text
    assert "| `attention` | `bf16`, `f16`, `f32` | `strided` | 2+ | yes | composed |" in text
    assert "| `broadcast` | — | `bf16`, `f16`, `f32` |" in text
