"""Shape rule of the attention descriptor and device detection of the C++ host mirror: the parts that need no
device (what ShapeRule::lower proves in the reference, and detect.rs:188-245's device-independent tests)."""
import pytest

from incin_amd import rocm_backend as RB
from incin_amd import rocm_exec as RX


def test_lowering_proves_the_output_shape():
    s = RX.AttentionSpec.lower((5, 8), (7, 8), (7, 6))
    assert s.out_dims == (5, 6) and s.group == 1
    s = RX.AttentionSpec.lower((2, 3, 40, 64), (2, 3, 72, 64), (2, 3, 72, 32), RB.BF16, causal=True)
    assert s.out_dims == (2, 3, 40, 32)
    # batch axes broadcast the NumPy way (cpu/ops/matmul.rs:198-221): [1,3,4]x[2,4,5] -> [2,3,5] carried over to attention
    s = RX.AttentionSpec.lower((1, 3, 4), (2, 6, 4), (2, 6, 5))
    assert s.out_dims == (2, 3, 5)
    s = RX.AttentionSpec.lower((2, 1, 3, 4), (1, 5, 7, 4), (1, 5, 7, 6))
    assert s.out_dims == (2, 5, 3, 6)
    # grouped queries: the last batch axis of q over 1 of k and v
    s = RX.AttentionSpec.lower((4, 8, 4, 16, 128), (4, 8, 1, 16, 128), (4, 8, 1, 16, 128), RB.BF16, causal=True, kv_lens=[16, 3, 0, 9])
    assert s.out_dims == (4, 8, 4, 16, 128) and s.group == 4


@pytest.mark.parametrize("args, fragment", [
    (((8,), (7, 8), (7, 8)), "rank >= 2"),
    (((5, 8), (7, 9), (7, 8)), "inner dims must match"),
    (((5, 8), (7, 8), (6, 8)), "key counts must match"),
    (((2, 5, 8), (3, 7, 8), (3, 7, 8)), "cannot broadcast"),
])
def test_lowering_refuses_what_the_operator_would_refuse(args, fragment):
    with pytest.raises(RB.BackendError) as e:
        RX.AttentionSpec.lower(*args)
    assert e.value.kind == "ShapeMismatch" and fragment in e.value.message
    assert "scaled_dot_product_attention" in e.value.message


def test_key_counts_are_checked_against_the_batch_axis():
    RX.AttentionSpec.lower((3, 4, 5, 8), (3, 4, 7, 8), (3, 4, 7, 8), kv_lens=[7, 0, 3])
    RX.AttentionSpec.lower((4, 5, 8), (4, 7, 8), (4, 7, 8), kv_lens=[6])            # below rank 4: one set of sequences
    for lens in ([7, 0], [7, 0, 3, 1]):
        with pytest.raises(RB.BackendError) as e:
            RX.AttentionSpec.lower((3, 4, 5, 8), (3, 4, 7, 8), (3, 4, 7, 8), kv_lens=lens)
        assert e.value.kind == "ShapeMismatch" and "key counts for a batch axis of 3" in e.value.message
    with pytest.raises(RB.BackendError) as e:
        RX.AttentionSpec.lower((3, 4, 5, 8), (3, 4, 7, 8), (3, 4, 7, 8), kv_lens=[7, 8, 3])
    assert "outside 0..=7" in e.value.message


def test_only_the_rocm_family_is_compiled_into_the_mirror():
    assert RX.is_compiled_in("rocm")
    for kind in ("cpu", "cuda", "wgpu", "metal"):
        assert not RX.is_compiled_in(kind)
        assert RX.probe(kind) is None                       # a family that is not compiled in is never detected


def test_detection_without_a_device_ends_on_the_cpu():
    # detect.rs:196-209: an empty preference still yields the CPU; a CPU-only preference yields the CPU
    assert RX.detect_device([]) == ("cpu", 0)
    assert RX.detect_device(["cpu"]) == ("cpu", 0)
    assert RX.detect_device(["cuda", "wgpu"]) == ("cpu", 0)
    kind, ordinal = RX.detect_device()
    assert kind in ("rocm", "cpu") and ordinal == 0
    assert RX.detect_device() == RX.detect_device()         # detection agrees with itself
