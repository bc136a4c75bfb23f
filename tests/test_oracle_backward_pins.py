"""Pins of the backward oracle (oracle/sdpa_backward.py).  The reference holds no value for attention gradients (its
gradient is whatever the tape walk gives), so the oracle is pinned by: the reference's hand-computed matmul
gradients (cpu/ops/matmul.rs:728-770), central differences of an independent float64 forward, closed forms, and
invariants a wrong sign, a dropped term or a transposed operand would break."""
import numpy as np
import pytest

from oracle import oracle as O
from oracle import sdpa_backward as BW


def rnd(seed, *shape):
    return np.random.Generator(np.random.PCG64(seed)).standard_normal(shape).astype(np.float32)


def test_matmul_rule_matches_the_reference_hand_computed_case():
    lhs = np.arange(1, 7, dtype=np.float32).reshape(2, 3)
    rhs = np.arange(7, 19, dtype=np.float32).reshape(3, 4)
    gl, gr = BW.matmul_backward(lhs, rhs, np.ones((2, 4), np.float32))
    assert gl.tolist() == [[34.0, 50.0, 66.0], [34.0, 50.0, 66.0]]
    assert gr.tolist() == [[5.0] * 4, [7.0] * 4, [9.0] * 4]


def loss(q, k, v, w, **kw):
    mask = None
    if kw.get("causal") or kw.get("kv_lens") is not None:
        b = np.broadcast_shapes(q.shape[:-2], k.shape[:-2], v.shape[:-2])
        mask = BW.additive_mask(q.shape[-2], k.shape[-2], b, kw.get("causal", False), kw.get("kv_lens"))
    if kw.get("mask") is not None:
        mask = kw["mask"] if mask is None else mask + kw["mask"]
    out = BW.sdpa_forward_f64(q, k, v, mask, kw.get("scale"))[0]
    return float((out * w).sum())


@pytest.mark.parametrize("case", [
    dict(q=(2, 5, 4), k=(2, 7, 4), v=(2, 7, 3)),
    dict(q=(2, 6, 4), k=(2, 6, 4), v=(2, 6, 4), causal=True),
    dict(q=(2, 3, 4), k=(2, 6, 4), v=(2, 6, 4), causal=True, scale=0.7),               # Sq != Skv: causal alignment
    dict(q=(3, 2, 4, 5, 8), k=(3, 2, 1, 6, 8), v=(3, 2, 1, 6, 8), causal=True),        # grouped queries: dk, dv sum over the group
    dict(q=(3, 1, 5, 4), k=(3, 1, 6, 4), v=(3, 1, 6, 4), kv_lens=np.array([6, 2, 4]).reshape(3, 1)),
    dict(q=(2, 5, 4), k=(2, 7, 4), v=(2, 7, 3), mask=True),
], ids=["plain", "causal", "causal_rect", "gqa", "kv_lens", "dense_mask"])
def test_gradients_match_central_differences(case):
    q, k, v = rnd(1, *case["q"]).astype(np.float64), rnd(2, *case["k"]).astype(np.float64), rnd(3, *case["v"]).astype(np.float64)
    kw = {n: case[n] for n in ("causal", "scale", "kv_lens") if n in case}
    if case.get("mask"):
        kw["mask"] = rnd(4, case["q"][-2], case["k"][-2]).astype(np.float64)
    out_shape = np.broadcast_shapes(q.shape[:-2], k.shape[:-2]) + (q.shape[-2], v.shape[-1])
    w = rnd(5, *out_shape).astype(np.float64)                   # loss = sum(out * w)  =>  grad_out = w
    dq, dk, dv = BW.sdpa_backward(q, k, v, w, **kw)
    r = np.random.Generator(np.random.PCG64(6))
    h = 1e-6
    for name, x, g in (("q", q, dq), ("k", k, dk), ("v", v, dv)):
        assert g.shape == x.shape
        for _ in range(12):
            idx = tuple(int(r.integers(0, n)) for n in x.shape)
            xp, xm = x.copy(), x.copy()
            xp[idx] += h
            xm[idx] -= h
            args = dict(q=q, k=k, v=v)
            fd = (loss(**{**args, name: xp}, w=w, **kw) - loss(**{**args, name: xm}, w=w, **kw)) / (2 * h)
            assert abs(fd - g[idx]) <= 1e-6 * max(1.0, abs(fd)), (name, idx, fd, g[idx])


def test_closed_forms():
    # one key: the softmax is 1 whatever q and k are, so dq = dk = 0 and dv = sum of the upstream rows
    q, k, v, go = rnd(1, 4, 3), rnd(2, 1, 3), rnd(3, 1, 5), rnd(4, 4, 5)
    dq, dk, dv = BW.sdpa_backward(q, k, v, go)
    assert np.abs(dq).max() == 0 and np.abs(dk).max() <= 1e-15
    assert np.allclose(dv, go.astype(np.float64).sum(0, keepdims=True), atol=1e-12)
    # scale 0: uniform weights 1/n; dv[j] = mean-weighted upstream, dq = dk = 0
    q, k, v, go = rnd(5, 4, 3), rnd(6, 6, 3), rnd(7, 6, 2), rnd(8, 4, 2)
    dq, dk, dv = BW.sdpa_backward(q, k, v, go, scale=0.0)
    assert np.abs(dq).max() == 0 and np.abs(dk).max() == 0
    assert np.allclose(dv, np.broadcast_to(go.astype(np.float64).sum(0) / 6, (6, 2)), atol=1e-12)
    # identical values: the output does not depend on the weights, so dq = dk = 0
    v1 = np.broadcast_to(rnd(9, 1, 2), (6, 2))
    dq, dk, dv = BW.sdpa_backward(q, k, v1, go)
    assert np.abs(dq).max() <= 1e-14 and np.abs(dk).max() <= 1e-14


def test_invariants():
    q, k, v, go = rnd(1, 2, 9, 8), rnd(2, 2, 9, 8), rnd(3, 2, 9, 8), rnd(4, 2, 9, 8)
    dq, dk, dv = BW.sdpa_backward(q, k, v, go, causal=True)
    # causal: the last key is seen by the last query only; key 0 by all
    p = BW.sdpa_forward_f64(q, k, v, BW.additive_mask(9, 9, (2,), True))[1]
    assert np.allclose(dv[:, 8], p[:, 8, 8, None] * go[:, 8], atol=1e-12)
    # total mass: sum_j dv_j = sum_i go_i (the weights of each row sum to one)
    assert np.allclose(dv.sum(1), go.astype(np.float64).sum(1), atol=1e-10)
    # permuting the keys permutes dk, dv and leaves dq
    perm = np.random.Generator(np.random.PCG64(9)).permutation(9)
    dq2, dk2, dv2 = BW.sdpa_backward(q, k[:, perm], v[:, perm], go)
    dq0, dk0, dv0 = BW.sdpa_backward(q, k, v, go)
    assert np.allclose(dq2, dq0, atol=1e-12) and np.allclose(dk2, dk0[:, perm], atol=1e-12) and np.allclose(dv2, dv0[:, perm], atol=1e-12)
    # padded keys get no gradient; the rest equals the truncated problem
    lens = np.array([9, 4]).reshape(2)
    dq3, dk3, dv3 = BW.sdpa_backward(q, k, v, go, kv_lens=lens.reshape(2, 1)[..., 0])
    assert np.abs(dk3[1, 4:]).max() == 0 and np.abs(dv3[1, 4:]).max() == 0
    dq4, dk4, dv4 = BW.sdpa_backward(q[1], k[1, :4], v[1, :4], go[1])
    assert np.allclose(dq3[1], dq4, atol=1e-12) and np.allclose(dk3[1, :4], dk4, atol=1e-12)


def test_forward_of_the_backward_oracle_is_the_forward_oracle():
    # the float64 forward used for the gradients agrees with the C restatement of the reference op
    q, k, v = rnd(1, 2, 3, 17, 16), rnd(2, 2, 3, 23, 16), rnd(3, 2, 3, 23, 8)
    a = BW.sdpa_forward_f64(q, k, v, BW.additive_mask(17, 23, (2, 3), True))[0]
    b = O.sdpa(q, k, v, causal=True)
    assert np.abs(a - b).max() <= 2e-6
    lse = BW.logsumexp(q, k, causal=True)
    x = np.einsum("bhid,bhjd->bhij", q.astype(np.float64), k.astype(np.float64)) * float(np.float32(0.25))
    x = x + BW.additive_mask(17, 23, (2, 3), True)
    assert np.allclose(lse, np.log(np.exp(x).sum(-1)), atol=1e-12)


def test_gradients_under_a_mask_that_widens_the_scores_match_central_differences():
    """q with one row under a mask of four rows and an extra leading axis: the gradient of the scores is summed back to the
    shape of q k^T before the first product's rules apply (cpu/tape.rs:243-265).  Checked by central differences."""
    r = np.random.Generator(np.random.PCG64(77))
    q, k, v = r.standard_normal((2, 3, 1, 8)), r.standard_normal((2, 1, 7, 8)), r.standard_normal((3, 7, 5))
    mask = r.standard_normal((5, 1, 1, 4, 7))
    g = r.standard_normal((5, 2, 3, 4, 5))
    dq, dk, dv = BW.sdpa_backward(q, k, v, g, mask=mask)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape

    def f(q_, k_, v_):
        return float((BW.sdpa_forward_f64(q_, k_, v_, mask)[0] * g).sum())

    eps = 1e-6
    for which, x, d in ((0, q, dq), (1, k, dk), (2, v, dv)):
        for _ in range(6):
            idx = tuple(int(r.integers(0, n)) for n in x.shape)
            xp, xm = x.copy(), x.copy()
            xp[idx] += eps
            xm[idx] -= eps
            args_p = [q, k, v]
            args_m = [q, k, v]
            args_p[which], args_m[which] = xp, xm
            num = (f(*args_p) - f(*args_m)) / (2 * eps)
            assert abs(num - d[idx]) < 1e-6 * max(1.0, abs(num)), (which, idx, num, d[idx])

