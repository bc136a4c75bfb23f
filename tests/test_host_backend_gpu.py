"""The attention op through the C++ host mirror of the reference's backend interface, written the way
the reference's own tests use the op (crates/incin/tests/medium_priority_ops_tests.rs:57-67:
storages in, optional mask and scale, storage out) and checked against the CPU oracle."""
import sys

import numpy as np
import pytest

from incin_amd import dtypes
from incin_amd import rocm_backend as RB
from oracle import oracle as O

pytestmark = pytest.mark.gpu
TOL = {RB.F32: 1e-5, RB.F16: 2e-2, RB.BF16: 2e-2}


def say(msg):
    print(msg, file=sys.stderr, flush=True)


def rnd(seed, shape, dtype):
    r = np.random.Generator(np.random.PCG64(seed))
    return dtypes.round_to(r.standard_normal(shape, dtype=np.float32), dtype)


def close(got, ref, tol, what):
    assert got.shape == ref.shape, "%s: shape %s vs %s" % (what, got.shape, ref.shape)
    nr = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nr), what + ": NaN pattern differs"
    err = float(np.abs(np.where(nr, 0, got) - np.where(nr, 0, ref)).max()) if got.size else 0.0
    say("%s: max-abs err %.3e" % (what, err))
    assert err <= tol, "%s: %.3e > %.0e" % (what, err, tol)


def test_ones_like_the_reference_test(gpu):
    # medium_priority_ops_tests.rs:57-67: ones [1,2,4] everywhere, no mask, default scale -> dims [1,2,4]
    say("host mirror: ones [1,2,4]")
    one = np.ones((1, 2, 4), np.float32)
    q, k, v = (RB.RocmStorage.from_numpy(one) for _ in range(3))
    attn = RB.scaled_dot_product_attention(q, k, v, None, None)
    assert attn.shape == (1, 2, 4)
    # softmax of equal scores is uniform, so the output is the mean of v's rows: all ones
    assert np.array_equal(attn.to_numpy(), one)


def test_bytes_round_trip_and_views(gpu):
    say("host mirror: from_bytes / to_bytes / views")
    a = rnd(1, (3, 4, 5), RB.F32)
    s = RB.RocmStorage.from_numpy(a)
    assert s.shape == (3, 4, 5)
    assert np.array_equal(s.to_numpy(), a)
    assert np.array_equal(s.transpose(0, 2).to_numpy(), a.transpose(2, 1, 0))
    assert np.array_equal(s.narrow(1, 1, 2).to_numpy(), a[:, 1:3])
    b = RB.RocmStorage.from_numpy(a[:, :1])
    assert np.array_equal(b.broadcast_as((2, 3, 4, 5)).to_numpy(), np.broadcast_to(a[:, :1], (2, 3, 4, 5)))
    h = rnd(2, (7, 9), RB.BF16)
    assert np.array_equal(RB.RocmStorage.from_numpy(h, RB.BF16).to_numpy(), h)
    with pytest.raises(RB.BackendError) as e:
        b.broadcast_as((3, 2, 4))
    assert e.value.kind == "ShapeMismatch"


@pytest.mark.parametrize("dtype", [RB.F32, RB.BF16, RB.F16])
@pytest.mark.parametrize("shape", [
    # (q shape, k shape, v shape)
    ((5, 8), (7, 8), (7, 6)),                                      # rank 2: one head, no batch axes
    ((3, 5, 16), (3, 9, 16), (3, 9, 16)),                          # rank 3
    ((2, 3, 40, 64), (2, 3, 72, 64), (2, 3, 72, 64)),              # [B, H, S, D]
    ((2, 6, 33, 64), (2, 1, 50, 64), (2, 1, 50, 64)),              # k, v broadcast over heads (one shared kv head)
    ((2, 2, 4, 130, 128), (2, 2, 1, 200, 128), (2, 2, 1, 200, 128)),     # grouped-query: q [B,Hkv,G,S,D], kv [B,Hkv,1,S,D]
    ((2, 1, 2, 3, 17, 32), (1, 2, 2, 1, 21, 32), (2, 2, 2, 1, 21, 32)),  # rank 6: leading axis looped on the host
], ids=["rank2", "rank3", "bhsd", "mqa_broadcast", "gqa5d", "rank6"])
def test_shapes_against_oracle(gpu, dtype, shape):
    qs, ks, vs = shape
    say("host mirror: q%s k%s v%s dtype %d" % (qs, ks, vs, dtype))
    q, k, v = rnd(10, qs, dtype), rnd(11, ks, dtype), rnd(12, vs, dtype)
    out = RB.scaled_dot_product_attention(RB.RocmStorage.from_numpy(q, dtype), RB.RocmStorage.from_numpy(k, dtype),
                                          RB.RocmStorage.from_numpy(v, dtype))
    ref = O.sdpa(q, k, v)
    assert out.dtype == dtype
    close(out.to_numpy(), ref, TOL[dtype], "shape %s" % (qs,))
    if len(qs) <= 5:
        assert RB.last_launch_count() == 1


@pytest.mark.parametrize("dtype", [RB.F32, RB.BF16])
def test_dense_masks_broadcast_like_the_reference(gpu, dtype):
    B, Hkv, G, Sq, Skv, D = 2, 2, 3, 37, 53, 64
    q, k, v = rnd(20, (B, Hkv, G, Sq, D), dtype), rnd(21, (B, Hkv, 1, Skv, D), dtype), rnd(22, (B, Hkv, 1, Skv, D), dtype)
    Q, K, V = (RB.RocmStorage.from_numpy(x, dtype) for x in (q, k, v))
    r = np.random.Generator(np.random.PCG64(23))
    for mshape in [(Sq, Skv), (1, Skv), (B, 1, 1, Sq, Skv), (B, Hkv, G, Sq, Skv), (1, Hkv, 1, Sq, 1), (B, Hkv, 1, 1, Skv)]:
        say("host mirror: dense mask %s dtype %d" % (mshape, dtype))
        m = dtypes.round_to(r.standard_normal(mshape, dtype=np.float32), dtype)
        m[r.random(mshape) < 0.2] = -np.inf
        m[..., 0] = 0.0                            # keep every row alive
        out = RB.scaled_dot_product_attention(Q, K, V, RB.RocmStorage.from_numpy(m, dtype), 0.3)
        close(out.to_numpy(), O.sdpa(q, k, v, mask=m, scale=0.3), TOL[dtype], "mask %s" % (mshape,))
    # a per-kv-head mask that is constant over the group cannot be folded into one head stride: the kv-head
    # axis is then looped on the host
    assert RB.last_launch_count() == Hkv
    # fully masked row -> NaN, as exp(log_softmax) of an all -inf row gives on the reference
    m = np.zeros((Sq, Skv), np.float32)
    m[5, :] = -np.inf
    out = RB.scaled_dot_product_attention(Q, K, V, RB.RocmStorage.from_numpy(m, dtype), None).to_numpy()
    assert np.isnan(out[:, :, :, 5]).all() and not np.isnan(np.delete(out, 5, axis=3)).any()


@pytest.mark.parametrize("dtype", [RB.F32, RB.BF16])
def test_tagged_masks_equal_their_dense_form(gpu, dtype):
    B, Hkv, G, Sq, Skv, D = 2, 2, 4, 96, 160, 128
    q, k, v = rnd(30, (B, Hkv, G, Sq, D), dtype), rnd(31, (B, Hkv, 1, Skv, D), dtype), rnd(32, (B, Hkv, 1, Skv, D), dtype)
    Q, K, V = (RB.RocmStorage.from_numpy(x, dtype) for x in (q, k, v))
    say("host mirror: causal tag dtype %d" % dtype)
    cm = O.causal_additive_mask(Sq, Skv)
    M = RB.RocmStorage.from_numpy(cm, dtype)
    dense = RB.scaled_dot_product_attention(Q, K, V, M).to_numpy()
    tagged = RB.scaled_dot_product_attention(Q, K, V, M.tag_causal()).to_numpy()
    ref = O.sdpa(q, k, v, mask=cm)
    close(dense, ref, TOL[dtype], "dense causal")
    close(tagged, ref, TOL[dtype], "tagged causal")
    say("host mirror: key-padding tag dtype %d" % dtype)
    lens = [160, 47]
    pm = np.zeros((B, 1, 1, 1, Skv), np.float32)
    for b, n in enumerate(lens):
        pm[b, ..., n:] = -np.inf
    P = RB.RocmStorage.from_numpy(pm, dtype)
    ref = O.sdpa(q, k, v, mask=pm)
    close(RB.scaled_dot_product_attention(Q, K, V, P).to_numpy(), ref, TOL[dtype], "dense padding")
    close(RB.scaled_dot_product_attention(Q, K, V, P.tag_key_padding(lens)).to_numpy(), ref, TOL[dtype], "tagged padding")


@pytest.mark.parametrize("dtype", [RB.F32, RB.BF16])
def test_mask_tags_read_off_the_mask(gpu, dtype):
    """infer_mask_tag: the causal mask as its callers build it, a key-padding mask and their sum are recognised from their
    rows (n zeros, then -inf) and tagged; anything else - values, a hole, a window, counts the tag cannot hold - comes back
    as it was.  A tagged mask gives what the tensor gives, forward and backward (where a mask tensor sends the gradients to
    the generic kernels and the tag does not)."""
    from oracle import sdpa_backward as BW
    B, H, Sq, Skv, D = 3, 2, 70, 100, 64
    q, k, v, go = rnd(60, (B, H, Sq, D), dtype), rnd(61, (B, H, Skv, D), dtype), rnd(62, (B, H, Skv, D), dtype), rnd(63, (B, H, Sq, D), dtype)
    S = lambda a: RB.RocmStorage.from_numpy(a, dtype)
    Q, K, V, GO = S(q), S(k), S(v), S(go)
    NEG = -np.inf
    causal = O.causal_additive_mask(Sq, Skv)                                   # [Sq, Skv], aligned to the last key
    pad = np.zeros((B, 1, 1, Skv), np.float32)
    for b, n in enumerate((100, 33, 71)):
        pad[b, ..., n:] = NEG
    both = causal[None, None] + pad
    cases = [("causal [Sq,Skv]", causal, 1), ("causal [1,1,Sq,Skv]", causal[None, None], 1), ("causal [H,Sq,Skv]", np.broadcast_to(causal, (H, Sq, Skv)).copy(), 1),
             ("key padding [B,1,1,Skv]", pad, 2), ("key padding [B,H,Sq,Skv]", np.broadcast_to(pad, (B, H, Sq, Skv)).copy(), 2),
             ("causal + key padding [B,1,Sq,Skv]", both, 3)]
    window = causal.copy()
    window[np.tril(np.ones((Sq, Skv), bool), Skv - Sq - 20)] = NEG             # a sliding window: rows start with -inf
    hole = causal.copy()
    hole[40, 3] = NEG
    values = causal.copy()
    values[10, 2] = -0.5
    one_padded = np.zeros((1, 1, 1, Skv), np.float32)
    one_padded[..., 50:] = NEG                                                 # one entry for a batch of unknown size: not tagged
    cases += [("window", window, 0), ("hole", hole, 0), ("values", values, 0), ("all zeros", np.zeros((Sq, Skv), np.float32), 0),
              ("one padded entry [1,1,1,Skv]", one_padded, 0), ("padding per head [H,1,Skv]", pad[:H, 0], 0)]
    tol = TOL[dtype]
    for what, m, kind in cases:
        say("host mirror: inferred mask tag, dtype %d: %s" % (dtype, what))
        M = S(np.ascontiguousarray(m))
        T, got_kind = M.infer_mask_tag()
        assert got_kind == kind, what
        assert T.shape == M.shape
        ref = O.sdpa(q, k, v, mask=m)
        close(RB.scaled_dot_product_attention(Q, K, V, T).to_numpy(), ref, tol, what)
        if kind == 0 and what not in ("window", "hole"):
            continue
        out, dq, dk, dv = RB.attention_backward(Q, K, V, GO, T)
        rq, rk, rv = BW.sdpa_backward(q, k, v, go, mask=m)
        gtol = 1e-5 if dtype == RB.F32 else 2e-2
        grad_close("dq " + what, dq.to_numpy(), rq, gtol)
        grad_close("dk " + what, dk.to_numpy(), rk, gtol)
        grad_close("dv " + what, dv.to_numpy(), rv, gtol)
    # a tag is kept, not inferred again; a view of a mask is read through its strides
    T, kind = S(causal).tag_causal().infer_mask_tag()
    assert kind == 0
    wide = np.full((Sq, Skv + 12), 7.0, np.float32)                            # a mask inside a wider buffer whose padding is not a mask
    wide[:, :Skv] = causal
    T, kind = S(wide).narrow(1, 0, Skv).infer_mask_tag()
    assert kind == 1


def test_key_lengths_with_one_shared_kv_head(gpu):
    # rank-4 multi-query layout: q [B,H,S,D] against k, v [B,1,S,D]; the key counts are per batch entry
    say("host mirror: multi-query operands with tagged key padding")
    dtype = RB.BF16
    B, H, Sq, Skv, D = 3, 4, 33, 150, 128
    q, k, v = rnd(45, (B, H, Sq, D), dtype), rnd(46, (B, 1, Skv, D), dtype), rnd(47, (B, 1, Skv, D), dtype)
    lens = [150, 1, 77]
    pm = np.zeros((B, 1, 1, Skv), np.float32)
    for b, n in enumerate(lens):
        pm[b, ..., n:] = -np.inf
    Q, K, V = (RB.RocmStorage.from_numpy(x, dtype) for x in (q, k, v))
    P = RB.RocmStorage.from_numpy(pm, dtype).tag_key_padding(lens)
    close(RB.scaled_dot_product_attention(Q, K, V, P).to_numpy(), O.sdpa(q, k, v, mask=pm), TOL[dtype], "multi-query padding")
    assert RB.last_launch_count() == 1


def test_views_as_operands(gpu):
    # k handed over as a narrowed, transposed-back view of a larger cache; q as a slice of a [B,S,H,D] layout
    say("host mirror: strided operands")
    dtype = RB.BF16
    B, H, S, D, CAP = 2, 4, 48, 64, 80
    q_bshd = rnd(40, (B, S, H, D), dtype)
    kc, vc = rnd(41, (B, H, CAP, D), dtype), rnd(42, (B, H, CAP, D), dtype)
    Q = RB.RocmStorage.from_numpy(q_bshd, dtype).transpose(1, 2)
    K = RB.RocmStorage.from_numpy(kc, dtype).narrow(2, 8, 60)
    V = RB.RocmStorage.from_numpy(vc, dtype).narrow(2, 8, 60)
    out = RB.scaled_dot_product_attention(Q, K, V)
    ref = O.sdpa(q_bshd.transpose(0, 2, 1, 3), kc[:, :, 8:68], vc[:, :, 8:68])
    close(out.to_numpy(), ref, TOL[dtype], "strided operands")


@pytest.mark.parametrize("dtype", [RB.F32, RB.BF16])
def test_operands_with_a_strided_last_axis(gpu, dtype):
    """k handed over as transpose(kt) of [.., D, Skv] storage - the view the reference's own matmul test goes through
    (cpu/ops/matmul.rs:677-724) - and v, q the same way, one of them also repeated over heads (stride 0): any view is an
    operand (cpu/storage.rs:308-325).  Checked against the oracle, whose strided arm reads the same views."""
    say("host mirror: operands whose last axis is strided, dtype %s" % dtype)
    B, H, Sq, Skv, D = 2, 3, 40, 70, 64
    q = rnd(60, (B, H, Sq, D), dtype)
    kt, vt = rnd(61, (B, 1, D, Skv), dtype), rnd(62, (B, H, D, Skv), dtype)        # stored transposed; k shared by the heads
    Q = RB.RocmStorage.from_numpy(q, dtype)
    K = RB.RocmStorage.from_numpy(kt, dtype).transpose(2, 3).broadcast_as((B, H, Skv, D))
    V = RB.RocmStorage.from_numpy(vt, dtype).transpose(2, 3)
    assert K.strides[-1] != 1 and V.strides[-1] != 1 and K.strides[1] == 0
    k_log = np.broadcast_to(kt.transpose(0, 1, 3, 2), (B, H, Skv, D))
    v_log = vt.transpose(0, 1, 3, 2)
    assert np.array_equal(K.to_numpy(), k_log) and np.array_equal(V.to_numpy(), v_log)        # the device-side gather itself
    ref = O.sdpa(q, k_log, v_log)                       # numpy views: the oracle walks the same strides
    out = RB.scaled_dot_product_attention(Q, K, V)
    close(out.to_numpy(), ref, TOL[dtype], "transposed k and v")
    # q strided too, with a dense mask and a causal tag on top
    qt = rnd(63, (B, H, D, Sq), dtype)
    Qt = RB.RocmStorage.from_numpy(qt, dtype).transpose(2, 3)
    m = np.where(np.random.Generator(np.random.PCG64(64)).random((Sq, Skv)) < 0.2, -np.inf, 0.0).astype(np.float32)
    m[:, 0] = 0.0
    out = RB.scaled_dot_product_attention(Qt, K, V, mask=RB.RocmStorage.from_numpy(m, dtype))
    close(out.to_numpy(), O.sdpa(qt.transpose(0, 1, 3, 2), k_log, v_log, mask=m), TOL[dtype], "transposed q, k, v with a mask")


@pytest.mark.parametrize("dtype", [RB.F32, RB.BF16])
def test_operands_repeated_along_the_last_axis(gpu, dtype):
    """q and v as broadcast_as([.., S, 1] -> [.., S, D]) views: the last axis has stride 0.  The reference takes any view
    (cpu/storage.rs:308-325); here the view is written out at its full extent before the launch."""
    say("host mirror: operands with a stride-0 last axis, dtype %s" % dtype)
    B, H, Sq, Skv, D = 2, 3, 33, 50, 64
    q1, v1 = rnd(70, (B, H, Sq, 1), dtype), rnd(71, (B, H, Skv, 1), dtype)
    k = rnd(72, (B, H, Skv, D), dtype)
    Q = RB.RocmStorage.from_numpy(q1, dtype).broadcast_as((B, H, Sq, D))
    V = RB.RocmStorage.from_numpy(v1, dtype).broadcast_as((B, H, Skv, D))
    K = RB.RocmStorage.from_numpy(k, dtype)
    assert Q.strides[-1] == 0 and V.strides[-1] == 0
    ref = O.sdpa(np.broadcast_to(q1, (B, H, Sq, D)), k, np.broadcast_to(v1, (B, H, Skv, D)))
    out = RB.scaled_dot_product_attention(Q, K, V)
    close(out.to_numpy(), ref, TOL[dtype], "q and v repeated along the last axis")
    # also repeated over the heads (two stride-0 axes, one of them the last)
    q2 = rnd(73, (B, 1, Sq, 1), dtype)
    Q2 = RB.RocmStorage.from_numpy(q2, dtype).broadcast_as((B, H, Sq, D))
    out = RB.scaled_dot_product_attention(Q2, K, V)
    close(out.to_numpy(), O.sdpa(np.broadcast_to(q2, (B, H, Sq, D)), k, np.broadcast_to(v1, (B, H, Skv, D))), TOL[dtype],
          "q repeated along heads and the last axis")


def test_decode_step(gpu):
    # one query token per head against a long cache: the split-KV path behind the same call
    say("host mirror: decode step")
    dtype = RB.BF16
    B, Hkv, G, Skv, D = 3, 2, 4, 3000, 128
    q, k, v = rnd(50, (B, Hkv, G, 1, D), dtype), rnd(51, (B, Hkv, 1, Skv, D), dtype), rnd(52, (B, Hkv, 1, Skv, D), dtype)
    out = RB.scaled_dot_product_attention(*(RB.RocmStorage.from_numpy(x, dtype) for x in (q, k, v)))
    close(out.to_numpy(), O.sdpa(q, k, v), TOL[dtype], "decode")


def test_empty_extents(gpu):
    say("host mirror: empty extents")
    q, k, v = np.zeros((2, 3, 4), np.float32), np.zeros((2, 0, 4), np.float32), np.zeros((2, 0, 5), np.float32)
    out = RB.scaled_dot_product_attention(*(RB.RocmStorage.from_numpy(x) for x in (q, k, v)))
    assert out.shape == (2, 3, 5) and np.array_equal(out.to_numpy(), np.zeros((2, 3, 5), np.float32))
    q0 = np.zeros((2, 0, 4), np.float32)
    k1, v1 = np.ones((2, 6, 4), np.float32), np.ones((2, 6, 5), np.float32)
    out = RB.scaled_dot_product_attention(*(RB.RocmStorage.from_numpy(x) for x in (q0, k1, v1)))
    assert out.shape == (2, 0, 5)


def test_error_behaviour(gpu):
    say("host mirror: error kinds")
    f = RB.RocmStorage.from_numpy
    q, k, v = f(np.ones((2, 4, 8), np.float32)), f(np.ones((2, 6, 8), np.float32)), f(np.ones((2, 6, 8), np.float32))

    def kind(*a, **kw):
        with pytest.raises(RB.BackendError) as e:
            RB.scaled_dot_product_attention(*a, **kw)
        return e.value.kind

    assert kind(q, f(np.ones((2, 6, 7), np.float32)), v) == "ShapeMismatch"          # q.D != k.D
    assert kind(q, k, f(np.ones((2, 5, 8), np.float32))) == "ShapeMismatch"          # k and v key counts differ
    assert kind(q, f(np.ones((3, 6, 8), np.float32)), f(np.ones((3, 6, 8), np.float32))) == "ShapeMismatch"   # batch 2 vs 3
    assert kind(f(np.ones((8,), np.float32)), k, v) == "ShapeMismatch"               # rank 1
    assert kind(q, k, v, f(np.ones((4, 5), np.float32))) == "ShapeMismatch"          # mask does not broadcast
    assert kind(q, f(np.ones((2, 6, 8), np.float32), RB.BF16), v) == "DTypeStorageMismatch"
    assert kind(q, k, v, f(np.zeros((4, 6), np.float32), RB.F16)) == "DTypeStorageMismatch"
    with pytest.raises(RB.BackendError) as e:
        RB.RocmStorage.from_numpy(np.ones(4, np.float32), device=99)
    assert e.value.kind == "InvalidDeviceOrdinal"
    with pytest.raises(RB.BackendError) as e:
        RB.RocmStorage.from_bytes(b"\0" * 8, (4,), 7)
    assert e.value.kind == "UnsupportedDType"
    with pytest.raises(RB.BackendError) as e:
        RB.RocmStorage.from_bytes(b"\0" * 8, (4,), RB.F32)
    assert e.value.kind == "Msg"
    # a head dimension beyond every kernel is a refusal, never a host fallback
    big = f(np.ones((2, 4, 300), np.float32))
    assert kind(big, big, big) == "UnsupportedBackendOperation"


# ---- gradients through the host mirror ------------------------------------------------------------------------------
def grad_close(name, got, ref, tol):
    ref = np.asarray(ref, np.float64)
    scale = float(np.abs(ref).max()) or 1.0
    err = float(np.abs(got - ref).max()) / scale
    say("   %s: max-abs err / max|ref| = %.3e" % (name, err))
    assert got.shape == ref.shape and err <= tol, "%s: %.3e" % (name, err)


@pytest.mark.parametrize("case", [
    # q shape, k shape, v shape, dtype, mask kind
    ((5, 8), (7, 8), (7, 6), RB.F32, None),                              # rank 2, the shape of the reference's matmul tests
    ((2, 3, 9, 16), (2, 3, 11, 16), (2, 3, 11, 16), RB.F32, "dense"),    # [B, H, S, D] with a dense mask
    ((2, 2, 4, 20, 128), (2, 2, 1, 20, 128), (2, 2, 1, 20, 128), RB.BF16, "causal"),    # grouped queries the reference's way
    ((3, 2, 2, 10, 32), (3, 2, 2, 12, 32), (3, 2, 2, 12, 32), RB.F32, None),            # an outer axis: one launch per index
    ((2, 6, 40, 128), (2, 1, 40, 128), (2, 1, 40, 128), RB.F16, "causal"),              # one shared kv head
], ids=["rank2", "dense_mask", "gqa_causal", "outer_axis", "shared_kv_head"])
def test_gradients_through_the_host_mirror(gpu, case):
    from oracle import sdpa_backward as BW
    qs, ks, vs, dtype, mk = case
    say("host mirror backward: %s" % (case,))
    q, k, v = rnd(41, qs, dtype), rnd(42, ks, dtype), rnd(43, vs, dtype)
    go = rnd(44, np.broadcast_shapes(qs[:-2], ks[:-2]) + (qs[-2], vs[-1]), dtype)
    Sq, Skv = qs[-2], ks[-2]
    mask_np, mask = None, None
    if mk == "dense":
        mask_np = rnd(45, (1, qs[1], Sq, Skv), dtype)
        mask_np[..., 3] = -np.inf
        mask = RB.RocmStorage.from_numpy(mask_np, dtype)
    elif mk == "causal":
        mask_np = np.triu(np.full((Sq, Skv), -np.inf, np.float32), 1 + Skv - Sq)
        mask = RB.RocmStorage.from_numpy(mask_np, dtype).tag_causal()
    S = lambda a: RB.RocmStorage.from_numpy(a, dtype)
    out, dq, dk, dv = RB.attention_backward(S(q), S(k), S(v), S(go), mask, None)
    assert dq.shape == qs and dk.shape == ks and dv.shape == vs
    rq, rk, rv = BW.sdpa_backward(q, k, v, go, mask=mask_np)
    tol = 1e-5 if dtype == RB.F32 else 2e-2
    grad_close("dq", dq.to_numpy(), rq, tol)
    grad_close("dk", dk.to_numpy(), rk, tol)
    grad_close("dv", dv.to_numpy(), rv, tol)
    ref = O.sdpa(q, k, v, mask=mask_np) if hasattr(O, "sdpa") else None
    if ref is not None:
        close(out.to_numpy(), ref, TOL[dtype], "forward beside the gradients")


@pytest.mark.parametrize("dtype", [RB.F32, RB.BF16])
@pytest.mark.parametrize("case", [
    ((3, 5, 16), (3, 7, 16), (3, 7, 8), (2, 1, 5, 7)),              # the mask adds a leading axis
    ((2, 3, 1, 16), (2, 3, 7, 16), (2, 3, 7, 16), (4, 7)),          # one query row, four mask rows
    ((1, 3, 5, 16), (1, 3, 7, 16), (1, 3, 7, 16), (4, 1, 1, 7)),    # an axis of extent 1 widened by the mask
    ((1, 16), (7, 16), (7, 8), (3, 2, 5, 7)),                       # rank-2 operands under a rank-4 mask
    ((2, 2, 4, 9, 64), (2, 2, 1, 11, 64), (2, 2, 1, 11, 64), (3, 1, 1, 1, 9, 11)),      # grouped queries under a mask with one more axis
], ids=["leading_axis", "rows", "widened_axis", "rank2", "gqa_leading_axis"])
def test_masks_that_widen_the_scores(gpu, dtype, case):
    """The reference adds the mask with a two-way broadcast (cpu/ops/shape_ops.rs:1262-1266, cpu/stride.rs:86-106): a mask
    with more leading axes, or more rows than q has, widens the scores and the output with them."""
    qs, ks, vs, msh = case
    say("host mirror: mask %s widens the scores of q %s, dtype %s" % (msh, qs, dtype))
    q, k, v = rnd(80, qs, dtype), rnd(81, ks, dtype), rnd(82, vs, dtype)
    mask = rnd(83, msh, dtype)
    mask[..., 2] = -np.inf
    S = lambda a: RB.RocmStorage.from_numpy(a, dtype)
    out = RB.scaled_dot_product_attention(S(q), S(k), S(v), mask=S(mask))
    ref = O.sdpa(q, k, v, mask=mask)
    assert out.shape == ref.shape
    close(out.to_numpy(), ref, TOL[dtype], "widening mask")
    # and its gradients: the widened axes are summed back (cpu/tape.rs:243-265)
    from oracle import sdpa_backward as BW
    go = rnd(84, ref.shape, dtype)
    out2, dq, dk, dv = RB.attention_backward(S(q), S(k), S(v), S(go), S(mask))
    assert dq.shape == qs and dk.shape == ks and dv.shape == vs
    rq, rk, rv = BW.sdpa_backward(q, k, v, go, mask=mask)
    tol = 1e-5 if dtype == RB.F32 else 2e-2
    grad_close("dq", dq.to_numpy(), rq, tol)
    grad_close("dk", dk.to_numpy(), rk, tol)
    grad_close("dv", dv.to_numpy(), rv, tol)
    close(out2.to_numpy(), ref, TOL[dtype], "forward beside the gradients")
    # a mask with more keys than k has would widen the scores past v's rows
    with pytest.raises(RB.BackendError) as e:
        RB.scaled_dot_product_attention(S(q), S(k[..., :1, :]), S(v[..., :1, :]), mask=S(mask))
    assert e.value.kind == "ShapeMismatch"


@pytest.mark.parametrize("case", [
    # q shape, k shape, v shape, dtype, causal tag
    ((2, 3, 4, 8), (1, 3, 5, 8), (1, 3, 5, 8), RB.F32, False),          # k, v shared by the batch entries
    ((2, 1, 6, 16), (2, 3, 5, 16), (2, 3, 5, 16), RB.F32, False),       # q shared by the heads
    ((2, 3, 4, 8), (5, 8), (5, 8), RB.F32, False),                      # k, v of lower rank
    ((2, 3, 4, 8), (2, 1, 5, 8), (2, 3, 5, 8), RB.F32, False),          # k shared by the heads, v not: no group axis
    ((3, 1, 2, 4, 20, 64), (1, 2, 2, 1, 20, 64), (1, 2, 2, 1, 20, 64), RB.BF16, True),      # grouped queries + two more broadcast axes
    ((2, 4, 40, 128), (1, 1, 40, 128), (1, 1, 40, 128), RB.BF16, True),  # one kv head for all batch entries (matrix-core kernels)
    ((4, 2, 33, 64), (1, 2, 47, 64), (4, 1, 47, 64), RB.F16, False),
], ids=["kv_shared_by_batch", "q_shared_by_heads", "kv_lower_rank", "k_only", "gqa_plus_outer", "one_kv_head_bf16", "mixed_f16"])
def test_gradients_of_broadcast_operands(gpu, case):
    """An operand repeated along a batch axis gets the sum of the gradients of its repetitions (cpu/tape.rs:243-265)."""
    from oracle import sdpa_backward as BW
    qs, ks, vs, dtype, causal = case
    say("host mirror backward with broadcast operands: %s" % (case,))
    q, k, v = rnd(51, qs, dtype), rnd(52, ks, dtype), rnd(53, vs, dtype)
    oshape = np.broadcast_shapes(qs[:-2], ks[:-2], vs[:-2]) + (qs[-2], vs[-1])
    go = rnd(54, oshape, dtype)
    Sq, Skv = qs[-2], ks[-2]
    S = lambda a: RB.RocmStorage.from_numpy(a, dtype)
    mask_np, mask = None, None
    if causal:
        mask_np = np.triu(np.full((Sq, Skv), -np.inf, np.float32), 1 + Skv - Sq)
        mask = S(mask_np).tag_causal()
    out, dq, dk, dv = RB.attention_backward(S(q), S(k), S(v), S(go), mask)
    assert out.shape == oshape and dq.shape == qs and dk.shape == ks and dv.shape == vs
    rq, rk, rv = BW.sdpa_backward(q, k, v, go, mask=mask_np)
    tol = 1e-5 if dtype == RB.F32 else 2e-2
    grad_close("dq", dq.to_numpy(), rq, tol)
    grad_close("dk", dk.to_numpy(), rk, tol)
    grad_close("dv", dv.to_numpy(), rv, tol)
    close(out.to_numpy(), O.sdpa(q, k, v, mask=mask_np), TOL[dtype], "forward beside the gradients")


@pytest.mark.parametrize("dtype", [RB.F32, RB.BF16])
def test_gradients_of_views(gpu, dtype):
    """Operands that are views: k repeated over the heads by broadcast_as (to the reference an operand of the view's
    shape: every repetition gets a gradient of its own), q transposed, and an upstream gradient that is a transposed view."""
    from oracle import sdpa_backward as BW
    B, H, Sq, Skv, D = 2, 3, 12, 17, 64
    q_t = rnd(90, (B, H, D, Sq), dtype)                   # q stored transposed
    k1, v = rnd(91, (B, 1, Skv, D), dtype), rnd(92, (B, H, Skv, D), dtype)
    go_t = rnd(93, (B, H, D, Sq), dtype)                  # the upstream gradient too
    S = lambda a: RB.RocmStorage.from_numpy(a, dtype)
    Q = S(q_t).transpose(2, 3)
    K = S(k1).broadcast_as((B, H, Skv, D))
    GO = S(go_t).transpose(2, 3)
    assert K.strides[1] == 0 and not GO.is_contiguous()
    out, dq, dk, dv = RB.attention_backward(Q, K, S(v), GO)
    q_log, k_log, go_log = q_t.transpose(0, 1, 3, 2), np.broadcast_to(k1, (B, H, Skv, D)), go_t.transpose(0, 1, 3, 2)
    rq, rk, rv = BW.sdpa_backward(q_log, np.ascontiguousarray(k_log), v, go_log)
    assert dq.shape == q_log.shape and dk.shape == (B, H, Skv, D) and dv.shape == v.shape
    tol = 1e-5 if dtype == RB.F32 else 2e-2
    grad_close("dq", dq.to_numpy(), rq, tol)
    grad_close("dk (one per repetition)", dk.to_numpy(), rk, tol)
    grad_close("dv", dv.to_numpy(), rv, tol)


def test_gradient_shape_errors(gpu):
    q, go = rnd(51, (2, 3, 4, 8), RB.F32), rnd(54, (2, 3, 4, 8), RB.F32)
    S = RB.RocmStorage.from_numpy
    with pytest.raises(RB.BackendError) as e:
        RB.attention_backward(S(q), S(rnd(55, (2, 3, 5, 8), RB.F32)), S(rnd(56, (2, 3, 5, 8), RB.F32)), S(go[:, :, :3]))
    assert e.value.kind == "ShapeMismatch"


# ---- buffers released in stream order; operators recorded into launch graphs ---------------------------------------------
def test_operators_do_not_allocate_once_the_pool_is_warm(gpu):
    """The operator drops its temporaries (gathered operands, workspaces, row normalisers) while its kernels still use them:
    they go back to the pool in stream order (cuda/storage.rs:171-177 is the reference's counterpart) and the same call,
    made again, is served from the pool without a single device allocation - with the same results."""
    B, H, Sq, Skv, D = 2, 3, 40, 4160, 64
    q, kt, v = rnd(60, (B, H, Sq, D), RB.BF16), rnd(61, (B, 1, D, Skv), RB.BF16), rnd(62, (B, H, Skv, D), RB.BF16)
    go = rnd(63, (B, H, Sq, D), RB.BF16)
    S = lambda a: RB.RocmStorage.from_numpy(a, RB.BF16)
    Q, V, GO = S(q), S(v), S(go)
    K = S(kt).transpose(2, 3).broadcast_as((B, H, Skv, D))              # gathered into a temporary by the operator
    outs = []
    for rep in range(3):
        before = RB.pool_stats()
        out = RB.scaled_dot_product_attention(Q, K, V)                   # (split launch: a workspace too)
        o2, dq, dk, dv = RB.attention_backward(Q, K, V, GO)
        after = RB.pool_stats()
        outs.append((out.to_numpy(), dq.to_numpy(), dk.to_numpy(), dv.to_numpy()))
        del out, o2, dq, dk, dv
        if rep == 2:
            assert after[0] == before[0], "device allocations on a warm pool: %r -> %r" % (before, after)
            assert after[1] > before[1]
    for a, b in zip(outs[0], outs[-1]):
        assert np.array_equal(a, b)
    k_log = np.broadcast_to(kt.transpose(0, 1, 3, 2), (B, H, Skv, D))
    close(outs[0][0], O.sdpa(q, k_log, v), TOL[RB.BF16], "forward on a warm pool")
    RB.trim_pool()
    assert RB.pool_stats()[2] == 0


def test_recorded_operator_with_a_transposed_k(gpu):
    """The operator with k handed over as a transposed view (gathered into a temporary first), recorded into a launch graph on
    a stream of the caller's and replayed: no step of it waits for the device or allocates while recording; every replay -
    with eager work on the same operands and synchronisations in between - gives what an eager call gives on the operands'
    current contents."""
    from incin_amd import capi
    B, H, Sq, Skv, D = 2, 4, 48, 300, 64
    dtype = RB.BF16
    q, kt, v = rnd(70, (B, H, Sq, D), dtype), rnd(71, (B, H, D, Skv), dtype), rnd(72, (B, H, Skv, D), dtype)
    S = lambda a: RB.RocmStorage.from_numpy(a, dtype)
    Q, Kt, V = S(q), S(kt), S(v)
    K = Kt.transpose(2, 3)
    stream = capi.Stream()
    RB.set_stream(stream.ptr)
    try:
        warm = RB.scaled_dot_product_attention(Q, K, V)                  # fills the pool with what the recording will ask for
        ref0 = warm.to_numpy()
        del warm
        with RB.Recording() as rec:
            out = RB.scaled_dot_product_attention(Q, K, V)
        stream.sync()
        k_log = kt.transpose(0, 1, 3, 2)
        close(ref0, O.sdpa(q, k_log, v), TOL[dtype], "eager call on the stream")
        for rep in range(4):
            # new contents for q, written in place; an eager call on the same operands between the replays
            q_new = rnd(80 + rep, (B, H, Sq, D), dtype)
            stream.sync()
            raw = dtypes.encode(q_new, dtype)
            capi.check(capi.load().incin_rocm_memcpy_h2d(0, Q.data_ptr, raw.ctypes.data, raw.nbytes))
            rec.replay()
            eager = RB.scaled_dot_product_attention(Q, K, V)
            got, want = out.to_numpy(), eager.to_numpy()                 # (to_bytes waits for the stream)
            assert np.array_equal(got, want), "replay %d differs from the eager call" % rep
            close(got, O.sdpa(q_new, k_log, v), TOL[dtype], "replay %d" % rep)
        rec.release()
    finally:
        RB.set_stream(None)
        stream.sync()
        stream.destroy()

