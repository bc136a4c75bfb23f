"""The conformance suite of the rocm backend mirror on a device (the reference runs the same suite against its CPU
adapter in crates/incin-backends/tests/conformance.rs), the attention descriptor's execution path against the CPU
oracle, and device detection with a device present."""
import sys

import numpy as np
import pytest

from incin_amd import dtypes
from incin_amd import rocm_backend as RB
from incin_amd import rocm_exec as RX
from oracle import oracle as O

pytestmark = pytest.mark.gpu
TOL = {RB.F32: 1e-5, RB.F16: 2e-2, RB.BF16: 2e-2}


def say(msg):
    print(msg, file=sys.stderr, flush=True)


def rnd(seed, shape, dtype):
    r = np.random.Generator(np.random.PCG64(seed))
    return dtypes.round_to(r.standard_normal(shape, dtype=np.float32), dtype)


def run_conformance(device=0):
    """The harness lives on the test side (tests/native/, built by `python -m incin_amd.build` beside the product
    libraries): its report in the reference's text form plus the three counts."""
    import collections
    import ctypes as C
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "libincin_rocm_conformance.so")
    assert os.path.exists(path), "tests/native/libincin_rocm_conformance.so is not built; run `python -m incin_amd.build`"
    RB.lib()                                            # the product libraries first: the harness links against them
    L = C.CDLL(path)
    L.incin_conformance_run.restype = C.c_size_t
    L.incin_conformance_run.argtypes = [C.c_int32, C.c_char_p, C.c_size_t] + [C.POINTER(C.c_int32)] * 3
    p, s, f = C.c_int32(), C.c_int32(), C.c_int32()
    buf = C.create_string_buffer(16384)
    L.incin_conformance_run(device, buf, len(buf), C.byref(p), C.byref(s), C.byref(f))
    return collections.namedtuple("Report", "text passed skipped failed")(buf.value.decode(), p.value, s.value, f.value)


def test_conformance_report(gpu):
    say("conformance suite on rocm:0")
    rep = run_conformance(0)
    say(rep.text)
    assert rep.failed == 0, rep.text
    lines = rep.text.splitlines()
    assert lines[0] == "conformance: rocm:0"
    # matmul is not registered, so its three checks are skips that carry the registry's reason - not passes
    assert rep.skipped == 3
    assert "  skip  matmul_is_within_tolerance (operation matmul is not registered)" in lines
    for name in ("storage_round_trips_its_values", "metadata_describes_the_tensor_it_came_from",
                 "reshape_preserves_element_order", "reshape_rejects_a_mismatched_operand",
                 "attention_is_within_tolerance", "attention_output_matches_its_descriptor",
                 "attention_rejects_a_wrong_input_count", "attention_descriptor_facts_equal_an_explicit_mask",
                 "attention_gradients_are_within_tolerance", "attention_gradients_have_their_operands_shapes",
                 "dispatch_routes_attention_to_the_holder_of_its_operands", "the_registry_and_the_executor_agree"):
        assert "  pass  " + name in lines, name
    assert rep.passed == 12


@pytest.mark.parametrize("dtype", [RB.F32, RB.BF16, RB.F16])
def test_descriptor_with_causal_and_key_counts_and_groups(gpu, dtype):
    # what a mask tensor cannot say compactly: causal alignment AND ragged key counts, on grouped queries
    B, Hkv, G, Sq, Skv, D = 3, 2, 4, 70, 130, 128
    lens = [130, 64, 7]
    say("descriptor path: q[%d,%d,%d,%d,%d] kv[%d,%d,1,%d,%d] causal, key counts %s, dtype %d" % (B, Hkv, G, Sq, D, B, Hkv, Skv, D, lens, dtype))
    q, k, v = rnd(1, (B, Hkv, G, Sq, D), dtype), rnd(2, (B, Hkv, 1, Skv, D), dtype), rnd(3, (B, Hkv, 1, Skv, D), dtype)
    spec = RX.AttentionSpec.lower(q.shape, k.shape, v.shape, dtype, causal=True, kv_lens=lens)
    assert spec.group == G and spec.out_dims == (B, Hkv, G, Sq, D)
    out = spec.execute(RB.RocmStorage.from_numpy(q, dtype), RB.RocmStorage.from_numpy(k, dtype), RB.RocmStorage.from_numpy(v, dtype))
    assert out.shape == spec.out_dims and out.dtype == dtype
    ref = O.sdpa(q, k, v, causal=True, kv_lens=np.asarray(lens, np.int32).reshape(B, 1, 1))
    got = out.to_numpy()
    nr = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nr)           # rows that see no key (count 7 < Skv - Sq + 1 ...) are NaN in both
    err = float(np.abs(np.where(nr, 0, got) - np.where(nr, 0, ref)).max())
    say("   max-abs err %.3e, %d NaN rows" % (err, int(nr.all(-1).sum())))
    assert err <= TOL[dtype]


def test_descriptor_padded_queries(gpu):
    # a padded self-attention batch: the same lengths for keys and queries; rows inside the lengths are what they
    # are without q_lens, bit for bit
    B, H, S, D = 3, 4, 300, 128
    lens = [300, 129, 1]
    q, k, v = rnd(8, (B, H, S, D), RB.BF16), rnd(9, (B, H, S, D), RB.BF16), rnd(10, (B, H, S, D), RB.BF16)
    sq, sk, sv = (RB.RocmStorage.from_numpy(x, RB.BF16) for x in (q, k, v))
    plain = RX.AttentionSpec.lower(q.shape, k.shape, v.shape, RB.BF16, causal=True, kv_lens=lens).execute(sq, sk, sv).to_numpy()
    got = RX.AttentionSpec.lower(q.shape, k.shape, v.shape, RB.BF16, causal=True, kv_lens=lens, q_lens=lens).execute(sq, sk, sv).to_numpy()
    ref = O.sdpa(q, k, v, causal=True, kv_lens=np.asarray(lens, np.int32).reshape(B, 1, 1))
    for b in range(B):
        n = lens[b]
        assert np.array_equal(got[b, :, :n], plain[b, :, :n])
        assert float(np.abs(got[b, :, :n] - ref[b, :, :n]).max()) <= TOL[RB.BF16]
    with pytest.raises(RB.BackendError) as e:
        RX.AttentionSpec.lower(q.shape, k.shape, v.shape, RB.BF16, q_lens=[300, 301, 0])
    assert e.value.kind == "ShapeMismatch" and "query count 301 outside 0..=300" in e.value.message


def test_descriptor_scale_and_views(gpu):
    q, k, v = rnd(4, (2, 3, 33, 64), RB.F32), rnd(5, (2, 3, 50, 64), RB.F32), rnd(6, (2, 3, 50, 64), RB.F32)
    spec = RX.AttentionSpec.lower(q.shape, k.shape, v.shape, RB.F32, scale=0.3)
    # k arrives as a view: stored [2, 50, 3, 64], heads and keys swapped back
    ks = RB.RocmStorage.from_numpy(np.ascontiguousarray(k.transpose(0, 2, 1, 3))).transpose(1, 2)
    out = spec.execute(RB.RocmStorage.from_numpy(q), ks, RB.RocmStorage.from_numpy(v))
    err = float(np.abs(out.to_numpy() - O.sdpa(q, k, v, scale=0.3)).max())
    say("descriptor path, scale 0.3, k as a view: max-abs err %.3e" % err)
    assert err <= 1e-5
    # the executor checks handles against the proof
    with pytest.raises(RB.BackendError) as e:
        spec.execute(RB.RocmStorage.from_numpy(q), ks)
    assert e.value.kind == "ShapeMismatch" and "3 operands" in e.value.message
    with pytest.raises(RB.BackendError) as e:
        spec.execute(RB.RocmStorage.from_numpy(q[:, :, :32]), ks, RB.RocmStorage.from_numpy(v))
    assert e.value.kind == "ShapeMismatch" and "validated descriptor" in e.value.message
    with pytest.raises(RB.BackendError) as e:
        spec.execute(RB.RocmStorage.from_numpy(q, RB.BF16), ks, RB.RocmStorage.from_numpy(v))
    assert e.value.kind == "DTypeStorageMismatch"


def test_reshape_keeps_element_order(gpu):
    a = rnd(7, (4, 6), RB.F32)
    s = RB.RocmStorage.from_numpy(a)
    assert np.array_equal(RX.reshape(s, (2, 3, 4)).to_numpy(), a.reshape(2, 3, 4))
    with pytest.raises(RB.BackendError) as e:
        RX.reshape(s, (5, 5))
    assert e.value.kind == "ShapeMismatch"
    # a view that is not dense is gathered into a dense copy first, as the reference's reshape does (cpu/storage.rs:407-440)
    assert np.array_equal(RX.reshape(s.transpose(0, 1), (24,)).to_numpy(), a.T.reshape(24))


def test_detection_finds_the_device(gpu):
    assert RX.probe("rocm") == 0
    assert RX.detect_device() == ("rocm", 0)                     # cuda is not compiled in, rocm comes next
    assert RX.detect_device(["cpu", "rocm"]) == ("cpu", 0) or RX.detect_device(["cpu", "rocm"]) == ("rocm", 0)
    assert RX.detect_device(["rocm"]) == ("rocm", 0)
    for _ in range(3):                                           # probing repeatedly is survivable and stable
        assert RX.probe("rocm") == 0
