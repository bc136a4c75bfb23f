"""Executes what the rocm capability table advertises, the way the reference's capability_matrix suite executes the
boundary cases of its CPU rules (crates/incin-backends/tests/capability_matrix.rs:222-330): every dtype x layout x
{min rank, max rank} of every rule runs on the device and matches the CPU oracle / the host data, and cells the
registry refuses are refused by the operator too, with the error kind the refusal names."""
import sys

import numpy as np
import pytest

from incin_amd import dtypes
from incin_amd import rocm_backend as RB
from incin_amd import rocm_capability as RC
from oracle import oracle as O

pytestmark = pytest.mark.gpu
CODE = {"f32": RB.F32, "f16": RB.F16, "bf16": RB.BF16}
TOL = {"f32": 1e-5, "f16": 2e-2, "bf16": 2e-2}
RULES = {}
for _r in RC.registrations("rocm"):
    RULES.setdefault(_r.operation, _r)          # the first (native) rule of an operation
ATTENTION_CELLS = [(r.implementation, layout) for r in RC.registrations("rocm") if r.operation == "attention" for layout in r.layouts]


def say(msg):
    print(msg, file=sys.stderr, flush=True)


def rnd(seed, shape, dtype):
    r = np.random.Generator(np.random.PCG64(seed))
    return dtypes.round_to(r.standard_normal(shape, dtype=np.float32), CODE[dtype])


def operand(a, dtype, layout):
    """Storage holding `a` in the given layout class: dense, or a view with dense rows carved out of a larger
    allocation (narrow along the row axis and, with batch axes, a transpose of two of them)."""
    if layout == "contiguous":
        return RB.RocmStorage.from_numpy(a, CODE[dtype])
    if layout == "strided":        # stored with the last two axes swapped, viewed back: the last axis is strided
        s = RB.RocmStorage.from_numpy(np.ascontiguousarray(np.swapaxes(a, -1, -2)), CODE[dtype]).transpose(a.ndim - 1, a.ndim - 2)
        assert s.shape == a.shape and s.strides[-1] != 1 and np.array_equal(s.to_numpy(), a)
        return s
    assert layout == "row-wise"
    if a.ndim >= 4:        # store with the first two batch axes swapped and 2 spare rows, view it back
        big = np.zeros(a.shape[:-2] + (a.shape[-2] + 2, a.shape[-1]), np.float32)
        big[..., 1:-1, :] = a
        s = RB.RocmStorage.from_numpy(np.ascontiguousarray(np.swapaxes(big, 0, 1)), CODE[dtype])
        s = s.transpose(0, 1)
    else:
        big = np.zeros(a.shape[:-2] + (a.shape[-2] + 2, a.shape[-1]), np.float32)
        big[..., 1:-1, :] = a
        s = RB.RocmStorage.from_numpy(big, CODE[dtype])
    s = s.narrow(a.ndim - 2, 1, a.shape[-2])
    assert s.shape == a.shape and np.array_equal(s.to_numpy(), a)
    return s


def shapes_of_rank(rank):
    """q, k, v shapes of that rank: rank 2 is one head; rank 8 has four leading axes the host loops over or folds."""
    if rank == 2:
        return (9, 32), (13, 32), (13, 32)
    lead = (1, 2, 1, 2)[: rank - 4] if rank > 4 else ()
    core = {3: ((3,), (3,)), 4: ((2, 3), (2, 3))}.get(rank, ((2, 2), (2, 2)))
    q = lead + core[0] + (17, 64)
    k = lead + core[1] + (29, 64)
    return q, k, k


@pytest.mark.parametrize("dtype", RULES["attention"].dtypes)
@pytest.mark.parametrize("level, layout", ATTENTION_CELLS)
@pytest.mark.parametrize("rank", [RULES["attention"].min_rank, RULES["attention"].max_rank])
def test_attention_rule_boundary_cases_execute(gpu, dtype, level, layout, rank):
    case = RC.CapabilityQuery("attention", dtype, layout, rank)
    assert RC.support("rocm", case).level == level
    qs, ks, vs = shapes_of_rank(rank)
    say("capability cell %s: q%s k%s" % (case, qs, ks))
    q, k, v = rnd(1, qs, dtype), rnd(2, ks, dtype), rnd(3, vs, dtype)
    out = RB.scaled_dot_product_attention(operand(q, dtype, layout), operand(k, dtype, layout), operand(v, dtype, layout))
    ref = O.sdpa(q, k, v)
    assert out.shape == ref.shape
    err = float(np.abs(out.to_numpy() - ref).max())
    say("   max-abs err %.3e" % err)
    assert err <= TOL[dtype]


@pytest.mark.parametrize("dtype", RULES["attention"].dtypes)
@pytest.mark.parametrize("level, layout", ATTENTION_CELLS)
@pytest.mark.parametrize("rank", [RULES["attention"].min_rank, 3, RULES["attention"].max_rank])
@pytest.mark.parametrize("shared", [False, True], ids=["own_batch", "broadcast_batch"])
def test_attention_rule_boundary_cases_train(gpu, dtype, level, layout, rank, shared):
    """The same cells with `training` set: the rule says yes, so the gradients come out and match the backward oracle
    (1e-5 of the largest gradient magnitude for f32, 2e-2 for the 16-bit types).  `broadcast_batch`: k and v have extent 1
    on a batch axis where q has more, and (from rank 5 on) q has extent 1 on another - operands the reference's matmul
    broadcasts, whose gradients are sums over the repetitions (cpu/tape.rs:243-265)."""
    from oracle import sdpa_backward as BW
    assert RULES["attention"].training
    case = RC.CapabilityQuery("attention", dtype, layout, rank, training=True)
    assert RC.support("rocm", case).level == level
    qs, ks, vs = shapes_of_rank(rank)
    if shared:
        if rank == 2:
            pytest.skip("rank 2 has no batch axis to share")
        wide = [a for a in range(rank - 2) if qs[a] > 1]
        ks = vs = tuple(1 if a == wide[0] else n for a, n in enumerate(ks))
        if len(wide) > 1:
            qs = tuple(1 if a == wide[-1] else n for a, n in enumerate(qs))
    say("capability cell %s: q%s k%s" % (case, qs, ks))
    q, k, v = rnd(1, qs, dtype), rnd(2, ks, dtype), rnd(3, vs, dtype)
    go = rnd(6, np.broadcast_shapes(qs[:-2], ks[:-2]) + (qs[-2], vs[-1]), dtype)
    out, dq, dk, dv = RB.attention_backward(operand(q, dtype, layout), operand(k, dtype, layout), operand(v, dtype, layout),
                                            RB.RocmStorage.from_numpy(go, CODE[dtype]))
    tol = 1e-5 if dtype == "f32" else 2e-2
    for name, got, ref in zip(("dq", "dk", "dv"), (dq, dk, dv), BW.sdpa_backward(q, k, v, go)):
        err = float(np.abs(got.to_numpy() - ref).max() / np.abs(ref).max())
        say("   %s: max-abs err / max|ref| %.3e" % (name, err))
        assert got.shape == ref.shape and err <= tol


@pytest.mark.parametrize("dtype", RULES["storage"].dtypes)
@pytest.mark.parametrize("rank", [RULES["storage"].min_rank, RULES["storage"].max_rank])
def test_storage_and_broadcast_rules_execute(gpu, dtype, rank):
    say("capability cells storage / broadcast %s rank %d" % (dtype, rank))
    shape = (2, 1, 2, 1, 3, 1, 2, 5)[8 - rank:] if rank else ()
    a = rnd(4, shape, dtype)
    s = RB.RocmStorage.from_numpy(a, CODE[dtype])
    assert s.shape == shape and np.array_equal(s.to_numpy(), a)                  # storage, contiguous
    if rank >= 2:
        t = s.transpose(rank - 1, rank - 2)                                       # storage family, strided view
        assert np.array_equal(t.to_numpy(), np.swapaxes(a, -1, -2))
        wide = tuple(3 if d == 1 else d for d in shape)
        assert np.array_equal(s.broadcast_as(wide).to_numpy(), np.broadcast_to(a, wide))     # broadcast
    else:
        assert np.array_equal(s.broadcast_as((2, 3)).to_numpy(), np.broadcast_to(a, (2, 3)))


def test_refused_cells_are_refused_by_the_operator_too(gpu):
    say("capability cells the registry refuses")
    q = rnd(5, (2, 8, 16), "f32")
    s = RB.RocmStorage.from_numpy(q)
    # layout `strided` (last axis not dense) is served through a dense temporary: composed, and it runs
    assert RC.support("rocm", RC.CapabilityQuery("attention", "f32", "strided", 3)).level == "composed"
    t = RB.RocmStorage.from_numpy(np.ascontiguousarray(np.swapaxes(q, -1, -2))).transpose(1, 2)
    assert np.abs(RB.scaled_dot_product_attention(t, s, s).to_numpy() - O.sdpa(q, q, q)).max() <= 1e-5
    # a reshape of that view is a gather followed by re-addressing
    assert np.array_equal(t.reshape((16, 8, 2)).to_numpy(), q.reshape(16, 8, 2))
    # rank 1: registry says Rank, operator ShapeMismatch
    assert RC.support("rocm", RC.CapabilityQuery("attention", "f32", "contiguous", 1)).reason == "Rank"
    with pytest.raises(RB.BackendError) as e:
        v1 = RB.RocmStorage.from_numpy(np.ones(16, np.float32))
        RB.scaled_dot_product_attention(v1, v1, v1)
    assert e.value.kind == "ShapeMismatch"
    # a dtype the storage rule does not list cannot be created
    assert RC.support("rocm", RC.CapabilityQuery("storage", "f64", "contiguous", 1)).reason == "DType"
    with pytest.raises(RB.BackendError) as e:
        RB.RocmStorage.from_bytes(b"\0" * 16, (2,), 3)
    assert e.value.kind == "UnsupportedDType"
