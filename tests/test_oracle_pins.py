"""Pins the CPU oracle (oracle/) before anything is compared against it.

Three kinds of pin, none of which restates the oracle's own formula:
  * the reference's own known-answer vectors (tests/golden/reference_vectors.json);
  * an independent float64 numpy evaluation on small shapes;
  * closed forms and invariants that a dropped term, wrong sign, wrong index or a
    transposed operand would break.
"""
import json
import os

import numpy as np
import pytest

from oracle import oracle as O

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


# ---- reference-held vectors ------------------------------------------------------

def test_reference_attention_heads():
    g = GOLD["attention_heads"]
    for case in g["cases"]:
        q = np.array(case["q"], np.float32).reshape(2, 1)
        k = np.array(case["k"], np.float32).reshape(2, 1)
        v = np.array(case["v"], np.float32).reshape(2, 1)
        out = O.sdpa(q, k, v, scale=g["scale"]).reshape(-1)
        assert np.abs(out - np.array(case["expected"])).max() <= g["tol"]
        # both heads at once through the batch axis, as the reference's gather test lays them out
    qs = np.array([c["q"] for c in g["cases"]], np.float32).reshape(2, 2, 1)
    ks = np.array([c["k"] for c in g["cases"]], np.float32).reshape(2, 2, 1)
    vs = np.array([c["v"] for c in g["cases"]], np.float32).reshape(2, 2, 1)
    out = O.sdpa(qs, ks, vs, scale=g["scale"]).reshape(-1)
    exp = np.array([c["expected"] for c in g["cases"]]).reshape(-1)
    assert np.abs(out - exp).max() <= g["tol"]


def test_reference_sdpa_ones_smoke():
    g = GOLD["sdpa_ones"]
    x = np.ones(g["shape"], np.float32)
    out = O.sdpa(x, x, x)
    assert list(out.shape) == g["expected_dims"]
    assert np.abs(out - g["expected_value"]).max() <= g["tol"]


def test_reference_softmax_known_answers():
    g = GOLD["softmax"]
    for case in g["cases"]:
        p = O.softmax_lastdim(np.array(case["x"], np.float32))
        assert np.all(np.isfinite(p))
        assert np.abs(p - np.array(case["expected"])).max() <= case["tol"]
    p = O.softmax_lastdim(np.array(g["rows_sum_to_one"], np.float32))
    assert np.abs(p.sum(axis=-1) - 1.0).max() <= g["rows_sum_tol"]
    p = O.softmax_lastdim(np.array(g["monotonic"], np.float32))
    assert p[0] < p[1] < p[2]
    # the same vectors through the attention op: with q = [1], k = x as a column and v = I,
    # scale 1, the output row IS softmax(x)
    for case in g["cases"]:
        x = np.array(case["x"], np.float32)
        out = O.sdpa(np.ones((1, 1), np.float32), x.reshape(-1, 1), np.eye(len(x), dtype=np.float32), scale=1.0)
        assert np.abs(out.reshape(-1) - np.array(case["expected"])).max() <= case["tol"]


def test_reference_log_softmax_known_answer():
    g = GOLD["log_softmax"]
    out = O.log_softmax_lastdim(np.array(g["x"], np.float32))
    assert np.all(np.isfinite(out))
    assert np.abs(out - np.array(g["expected"])).max() <= g["tol"]


def test_reference_matmul_known_answers():
    for case in GOLD["matmul"]["cases"]:
        lhs = np.array(case["lhs"], np.float32)
        rhs = np.array(case["rhs"], np.float32)
        exp = np.array(case["expected"], np.float32)
        assert np.array_equal(O.gemm(lhs, rhs), exp)                       # FMA row-streaming arm
        assert np.array_equal(O.gemm(lhs, rhs, host_has_fma=False), exp)   # mul-then-add arm
        assert np.array_equal(O.gemm(lhs, np.asfortranarray(rhs)), exp)    # strided rhs: f64-accumulate arm
        lhs_t = np.ascontiguousarray(lhs.T).T                               # transposed (non-contiguous) lhs view
        assert not lhs_t.flags["C_CONTIGUOUS"]
        assert np.array_equal(O.gemm(lhs_t, rhs), exp)


def test_reference_batch_broadcast_shapes():
    r = rng(1)
    for case in GOLD["batch_broadcast_shapes"]["cases"]:
        # the reference pins matmul [..,M,K] x [..,K,N]; through attention that is q [..,M,K], k [..,N,K]
        lhs, rhs, out = case["lhs"], case["rhs"], case["out"]
        q = r.standard_normal(lhs, dtype=np.float32)
        k = r.standard_normal(rhs[:-2] + [rhs[-1], rhs[-2]], dtype=np.float32)
        v = r.standard_normal(rhs[:-2] + [rhs[-1], 7], dtype=np.float32)
        o = O.sdpa(q, k, v)
        assert list(o.shape) == out[:-1] + [7]
        assert np.abs(o - O.brute_f64(q, k, v)).max() < 1e-6
    assert O.broadcast_shape([2, 1, 3], [5, 1]) == [2, 5, 3]
    with pytest.raises(ValueError):
        O.broadcast_shape([2, 3], [4, 3])


# ---- a mask whose broadcast widens the scores (cpu/ops/shape_ops.rs:1262-1266, cpu/stride.rs:86-106) ----------------

@pytest.mark.parametrize("case", [
    ((3, 5, 8), (3, 7, 8), (3, 7, 6), (2, 1, 5, 7)),          # leading mask axis: the output gains it
    ((2, 3, 1, 8), (2, 3, 7, 8), (2, 3, 7, 8), (4, 7)),      # one query row, four mask rows: four output rows
    ((1, 3, 5, 8), (1, 3, 7, 8), (1, 3, 7, 8), (4, 1, 1, 7)),  # an axis of extent 1 widened by the mask
    ((1, 8), (7, 8), (7, 4), (3, 2, 5, 7)),                  # rank-2 operands under a rank-4 mask
], ids=["leading_axis", "rows", "widened_axis", "rank2"])
def test_mask_that_widens_the_scores(case):
    """The oracle against an independent float64 numpy evaluation, where numpy's own broadcasting does the widening, and
    against the same call with the operands widened by hand (which takes the ordinary path)."""
    from oracle import sdpa_backward as BW
    qs, ks, vs, msh = case
    r = rng(sum(qs) + sum(msh))
    q, k, v = (r.standard_normal(sh, dtype=np.float32) for sh in (qs, ks, vs))
    mask = r.standard_normal(msh, dtype=np.float32)
    mask[..., 2] = -np.inf
    got = O.sdpa(q, k, v, mask=mask)
    ref = BW.sdpa_forward_f64(q, k, v, mask)[0]
    assert got.shape == ref.shape
    assert np.abs(got - ref).max() < 1e-6
    rows = max(qs[-2], msh[-2] if len(msh) >= 2 else 1)
    bshape = np.broadcast_shapes(qs[:-2], ks[:-2], vs[:-2], msh[:-2])
    wide = O.sdpa(np.ascontiguousarray(np.broadcast_to(q, bshape + (rows, qs[-1]))), k, v, mask=mask)
    assert np.array_equal(got, wide)
    assert np.array_equal(got, O.sdpa_materialised(q, k, v, mask=mask))


# ---- independent float64 evaluation ---------------------------------------------------

@pytest.mark.parametrize("shape", [(1, 1, 8, 4), (2, 4, 64, 32), (1, 3, 17, 5), (2, 2, 33, 16)])
@pytest.mark.parametrize("masked", [False, True])
def test_against_float64_numpy(shape, masked):
    r = rng(hash(shape) % 1000 + masked)
    b, h, s, d = shape
    q = r.standard_normal(shape, dtype=np.float32)
    k = r.standard_normal((b, h, s + 3, d), dtype=np.float32)
    v = r.standard_normal((b, h, s + 3, d + 1), dtype=np.float32)
    mask = None
    if masked:
        mask = np.where(r.random((s, s + 3)) < 0.3, -np.inf, 0.0).astype(np.float32)
        mask[:, 0] = 0.0
        mask = mask + r.standard_normal((s, s + 3), dtype=np.float32) * 0.5
    got = O.sdpa(q, k, v, mask=mask)
    ref = O.brute_f64(q, k, v, mask=mask)
    assert np.abs(got - ref).max() < 1e-6
    assert np.array_equal(got, O.sdpa_materialised(q, k, v, mask=mask))


def test_row_streaming_and_materialised_forms_agree_bitwise():
    r = rng(7)
    q = r.standard_normal((2, 2, 3, 40, 16), dtype=np.float32)
    k = r.standard_normal((2, 2, 1, 50, 16), dtype=np.float32)
    v = r.standard_normal((2, 2, 1, 50, 24), dtype=np.float32)
    lens = np.array([13, 50], np.int32).reshape(2, 1, 1)
    a = O.sdpa(q, k, v, causal=True, kv_lens=lens)
    b = O.sdpa_materialised(q, k, v, causal=True, kv_lens=lens)
    assert np.array_equal(a, b, equal_nan=True)
    rows = np.array([[0, 0], [5, 39], [11, 20]])
    sel = O.sdpa_rows(q, k, v, rows, causal=True, kv_lens=lens)
    flat = a.reshape(-1, 40, 24)
    for n, (bi, i) in enumerate(rows):
        assert np.array_equal(sel[n], flat[bi, i], equal_nan=True)


# ---- closed forms and invariants ---------------------------------------------------------

def _qkv(seed, b=2, h=3, sq=24, skv=24, d=16, dv=16):
    r = rng(seed)
    return (r.standard_normal((b, h, sq, d), dtype=np.float32),
            r.standard_normal((b, h, skv, d), dtype=np.float32),
            r.standard_normal((b, h, skv, dv), dtype=np.float32))


def test_default_scale_is_inverse_sqrt_of_q_last_dim():
    q, k, v = _qkv(11, d=16)
    assert np.array_equal(O.sdpa(q, k, v), O.sdpa(q, k, v, scale=0.25))
    assert not np.array_equal(O.sdpa(q, k, v), O.sdpa(q, k, v, scale=1.0))


def test_scale_zero_gives_column_means_and_prefix_means():
    q, k, v = _qkv(12)
    out = O.sdpa(q, k, v, scale=0.0)
    assert np.abs(out - v.mean(axis=2, keepdims=True)).max() < 1e-6
    out = O.sdpa(q, k, v, scale=0.0, causal=True)
    prefix = np.cumsum(v.astype(np.float64), axis=2) / np.arange(1, v.shape[2] + 1)[None, None, :, None]
    assert np.abs(out - prefix).max() < 1e-6


def test_causal_first_row_is_first_value_row():
    q, k, v = _qkv(13)
    out = O.sdpa(q, k, v, causal=True)
    assert np.abs(out[:, :, 0] - v[:, :, 0]).max() < 1e-6


def test_dominant_key_selects_its_value_row():
    q, k, v = _qkv(14)
    mask = np.zeros((24, 24), np.float32)
    mask[np.arange(24), (np.arange(24) * 7) % 24] = 1e4
    out = O.sdpa(q, k, v, mask=mask)
    assert np.abs(out - v[:, :, (np.arange(24) * 7) % 24]).max() < 1e-6


def test_key_permutation_invariance_and_row_shift_invariance():
    q, k, v = _qkv(15)
    perm = rng(99).permutation(24)
    a = O.sdpa(q, k, v)
    b = O.sdpa(q, k[:, :, perm], v[:, :, perm])
    assert np.abs(a - b).max() < 2e-6
    shift = rng(98).standard_normal((24, 1)).astype(np.float32)
    c = O.sdpa(q, k, v, mask=np.broadcast_to(shift, (24, 24)))
    assert np.abs(a - c).max() < 2e-6


def test_output_rows_lie_in_convex_hull_of_values():
    q, k, v = _qkv(16)
    out = O.sdpa(q, k, v)
    assert np.all(out <= v.max(axis=2, keepdims=True) + 1e-6)
    assert np.all(out >= v.min(axis=2, keepdims=True) - 1e-6)


def test_transposed_operands_are_detected():
    # q k^T vs q^T k: with Sq != Skv != D a transposed operand changes the shape or the values
    r = rng(17)
    q = r.standard_normal((5, 3), dtype=np.float32)
    k = r.standard_normal((7, 3), dtype=np.float32)
    v = r.standard_normal((7, 2), dtype=np.float32)
    out = O.sdpa(q, k, v, scale=1.0)
    s = q.astype(np.float64) @ k.astype(np.float64).T
    p = np.exp(s - s.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    assert out.shape == (5, 2)
    assert np.abs(out - p @ v).max() < 1e-6


def test_decode_equals_last_row_of_causal_prefill():
    q, k, v = _qkv(18, sq=24, skv=24)
    full = O.sdpa(q, k, v, causal=True)
    last = O.sdpa(q[:, :, -1:], k, v, causal=True)          # Sq = 1: causal alignment puts it on the last key
    assert np.abs(full[:, :, -1:] - last).max() < 1e-6
    assert np.array_equal(last, O.sdpa(q[:, :, -1:], k, v))


def test_gqa_equals_mha_with_repeated_kv_heads():
    r = rng(19)
    q = r.standard_normal((2, 2, 3, 10, 8), dtype=np.float32)       # [B, Hkv, G, S, D]
    k = r.standard_normal((2, 2, 1, 12, 8), dtype=np.float32)
    v = r.standard_normal((2, 2, 1, 12, 8), dtype=np.float32)
    a = O.sdpa(q, k, v)
    b = O.sdpa(q, np.repeat(k, 3, axis=2), np.repeat(v, 3, axis=2))
    assert np.array_equal(a, b)


def test_padded_keys_equal_truncated_keys_and_causal_mask_construction():
    q, k, v = _qkv(20, sq=12, skv=20)
    lens = np.array([7, 20], np.int32).reshape(2, 1)
    a = O.sdpa(q, k, v, kv_lens=lens)
    assert np.array_equal(a[0], O.sdpa(q[0], k[0, :, :7], v[0, :, :7]))
    assert np.array_equal(a[1], O.sdpa(q[1], k[1], v[1]))
    m = O.causal_additive_mask(12, 20)
    assert m[0, 8] == 0.0 and m[0, 9] == -np.inf and m[11, 19] == 0.0
    assert np.array_equal(O.sdpa(q, k, v, mask=m), O.sdpa(q, k, v, causal=True))
    # triu as the reference evaluates it: keeps col >= row + k, zero elsewhere
    t = O.triu(np.arange(1, 10, dtype=np.float32).reshape(3, 3), 1)
    assert np.array_equal(t, np.array([[0, 2, 3], [0, 0, 6], [0, 0, 0]], np.float32))


def test_fully_masked_row_is_nan_and_nan_logit_poisons_row():
    q, k, v = _qkv(21, b=1, h=1, sq=4, skv=6)
    mask = np.zeros((4, 6), np.float32)
    mask[2, :] = -np.inf
    out = O.sdpa(q, k, v, mask=mask)
    assert np.all(np.isnan(out[0, 0, 2])) and np.all(np.isfinite(out[0, 0, [0, 1, 3]]))
    out = O.sdpa(q, k, v, kv_lens=np.array([0], np.int32).reshape(1, 1))
    assert np.all(np.isnan(out))
    mask = np.zeros((4, 6), np.float32)
    mask[1, 3] = np.nan
    out = O.sdpa(q, k, v, mask=mask)
    assert np.all(np.isnan(out[0, 0, 1])) and np.all(np.isfinite(out[0, 0, 0]))


def test_strided_views_take_the_same_values():
    q, k, v = _qkv(22, b=1, h=2, sq=9, skv=11, d=8, dv=8)
    kt = np.ascontiguousarray(np.swapaxes(k, -1, -2))      # stored as [.., D, Skv]; k is then a strided view
    k_view = np.swapaxes(kt, -1, -2)
    assert not k_view.flags["C_CONTIGUOUS"]
    a, b = O.sdpa(q, k, v), O.sdpa(q, k_view, v)
    assert np.abs(a - b).max() < 1e-6                        # different matmul arm (row-streaming), same values to rounding
    vt = np.swapaxes(np.ascontiguousarray(np.swapaxes(v, -1, -2)), -1, -2)
    assert np.abs(a - O.sdpa(q, k, vt)).max() < 1e-6
