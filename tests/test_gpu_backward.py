"""Attention backward through the C ABI against the backward oracle (the gradients the reference's tape walk
gives, oracle/sdpa_backward.py): dq, dk, dv for f16 / bf16 operands, D = 128, grouped queries, causal masks with
Sq != Skv, ragged key counts.  Tolerance: 2e-2 relative to the largest magnitude of the gradient tensor compared
(bf16 / f16 inputs, bf16 / f16 probabilities and dS as matrix operands, f32 accumulation)."""
import sys

import numpy as np
import pytest

from incin_amd import capi, dtypes, host
from oracle import sdpa_backward as BW

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, file=sys.stderr, flush=True)


def make(seed, B, Hq, Hkv, Sq, Skv, D, dtype):
    r = np.random.Generator(np.random.PCG64(seed))
    mk = lambda *s: dtypes.round_to(r.standard_normal(s, dtype=np.float32), dtype)
    return mk(B, Hq, Sq, D), mk(B, Hkv, Skv, D), mk(B, Hkv, Skv, D), mk(B, Hq, Sq, D)


def compare(name, got, ref, tol=2e-2):
    ref = np.asarray(ref, np.float64)
    scale = float(np.abs(ref).max()) or 1.0
    err = float(np.abs(got - ref).max()) / scale
    say("   %s: max-abs err / max|ref| = %.3e (max|ref| %.3g)" % (name, err, scale))
    assert not np.isnan(got).any(), name
    assert err <= tol, "%s: %.3e" % (name, err)


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, causal, kv_lens
    (1, 1, 1, 32, 32, False, None),
    (1, 1, 1, 128, 128, True, None),
    (2, 4, 4, 200, 333, False, None),
    (2, 4, 2, 300, 300, True, None),
    (1, 8, 2, 130, 450, True, None),                  # Sq < Skv: causal alignment, grouped queries
    (3, 2, 2, 257, 257, True, [257, 100, 31]),
    (2, 2, 1, 64, 700, False, [700, 1]),
], ids=["tiny", "one_tile_causal", "rect", "gqa_causal", "gqa_rect_causal", "ragged_causal", "ragged"])
@pytest.mark.parametrize("D", [128, 64])
def test_backward_against_the_oracle(gpu, dtype, shape, D):
    B, Hq, Hkv, Sq, Skv, causal, lens = shape
    G = Hq // Hkv
    say("backward: %s D=%d dtype %d" % (shape, D, dtype))
    q, k, v, go = make(11, B, Hq, Hkv, Sq, Skv, D, dtype)
    lens_a = None if lens is None else np.asarray(lens, np.int32)
    out, dq, dk, dv = host.sdpa_backward(q, k, v, go, dtype, causal=causal, kv_lens=lens_a)
    rq, rk, rv = BW.sdpa_backward(q.reshape(B, Hkv, G, Sq, D), k[:, :, None], v[:, :, None], go.reshape(B, Hkv, G, Sq, D),
                                  causal=causal, kv_lens=None if lens is None else lens_a.reshape(B, 1, 1))
    compare("dq", dq, rq.reshape(B, Hq, Sq, D))
    compare("dk", dk, rk.reshape(B, Hkv, Skv, D))
    compare("dv", dv, rv.reshape(B, Hkv, Skv, D))
    if lens is not None:
        for b in range(B):
            assert not dk[b, :, lens[b]:].any() and not dv[b, :, lens[b]:].any()      # padded keys: exactly zero


def test_backward_random_cases(gpu):
    """Seeded random shapes: batch, heads, group size, lengths on either side of the 64-row tiles and the 128-key
    workgroups, causal alignment with Sq <= Skv, ragged key counts >= 1 (every query row keeps a visible key, so the
    oracle has no NaN), scales.  Each case is printed before it runs."""
    r = np.random.Generator(np.random.PCG64(2026))
    for case in range(28):
        D = 128 if case % 3 else 64
        B, Hkv, G = int(r.integers(1, 4)), int(r.integers(1, 4)), int(r.choice([1, 2, 4]))
        Skv = int(r.choice([r.integers(1, 70), r.integers(60, 140), r.integers(120, 420)]))
        causal = bool(r.integers(0, 2))
        Sq = int(r.integers(1, Skv + 1)) if causal else int(r.integers(1, 300))
        lens = None
        if r.integers(0, 2):
            lens = r.integers(1, Skv + 1, B).astype(np.int32)      # (row 0 sees key 0 whenever Sq <= Skv and the count is >= 1)
        dtype = capi.BF16 if case % 2 else capi.F16
        scale = float(r.choice([0.0883883461356163, 0.05, 0.2]))
        Hq = Hkv * G
        say("backward random case %d: B=%d Hq=%d Hkv=%d Sq=%d Skv=%d causal=%s lens=%s dtype=%d scale=%g"
            % (case, B, Hq, Hkv, Sq, Skv, causal, None if lens is None else lens.tolist(), dtype, scale))
        q, k, v, go = make(100 + case, B, Hq, Hkv, Sq, Skv, D, dtype)
        out, dq, dk, dv = host.sdpa_backward(q, k, v, go, dtype, scale=scale, causal=causal, kv_lens=lens)
        rq, rk, rv = BW.sdpa_backward(q.reshape(B, Hkv, G, Sq, D), k[:, :, None], v[:, :, None], go.reshape(B, Hkv, G, Sq, D),
                                      scale=scale, causal=causal, kv_lens=None if lens is None else lens.reshape(B, 1, 1))
        rq, rk, rv = rq.reshape(B, Hq, Sq, D), rk.reshape(B, Hkv, Skv, D), rv.reshape(B, Hkv, Skv, D)
        assert not np.isnan(rq).any(), "case construction: a row without keys"
        compare("dq", dq, rq)
        compare("dk", dk, rk)
        compare("dv", dv, rv)


def test_backward_random_cases_f32(gpu):
    """The same draw in f32 over longer sequences: key and query counts up to 1600, where a call this small has the walks of
    its blocks dealt to 2 or 4 workgroups and its dQ kernel on a second stream - by the library's own rule, nothing forced.
    1e-5 of the largest gradient magnitude against the f64 oracle."""
    r = np.random.Generator(np.random.PCG64(2027))
    for case in range(18):
        D = 128 if case % 3 else 64
        B, Hkv, G = int(r.integers(1, 3)), int(r.integers(1, 4)), int(r.choice([1, 2, 4]))
        Skv = int(r.choice([r.integers(1, 140), r.integers(120, 700), r.integers(500, 1600), r.integers(1000, 1600)]))
        causal = bool(r.integers(0, 2))
        Sq = int(r.integers(1, Skv + 1)) if causal else int(r.choice([r.integers(1, 300), r.integers(500, 1300)]))
        lens = None
        if r.integers(0, 2):
            lens = r.integers(1, Skv + 1, B).astype(np.int32)
        scale = float(r.choice([1.0 / np.sqrt(D), 0.05, 0.2]))
        Hq = Hkv * G
        say("backward random case %d (f32): B=%d Hq=%d Hkv=%d Sq=%d Skv=%d D=%d causal=%s lens=%s scale=%g"
            % (case, B, Hq, Hkv, Sq, Skv, D, causal, None if lens is None else lens.tolist(), scale))
        q, k, v, go = make(300 + case, B, Hq, Hkv, Sq, Skv, D, capi.F32)
        out, dq, dk, dv = host.sdpa_backward(q, k, v, go, capi.F32, scale=scale, causal=causal, kv_lens=lens)
        rq, rk, rv = BW.sdpa_backward(q.reshape(B, Hkv, G, Sq, D), k[:, :, None], v[:, :, None], go.reshape(B, Hkv, G, Sq, D),
                                      scale=scale, causal=causal, kv_lens=None if lens is None else lens.reshape(B, 1, 1))
        rq, rk, rv = rq.reshape(B, Hq, Sq, D), rk.reshape(B, Hkv, Skv, D), rv.reshape(B, Hkv, Skv, D)
        assert not np.isnan(rq).any(), "case construction: a row without keys"
        compare("dq", dq, rq, tol=1e-5)
        compare("dk", dk, rk, tol=1e-5)
        compare("dv", dv, rv, tol=1e-5)


def test_rows_without_visible_keys_get_zero_gradients(gpu):
    # Sq > Skv under causal alignment: the first Sq - Skv rows see nothing (NaN in the forward).  They get a zero dq
    # and contribute nothing to dk, dv; the other rows are what the oracle gives for them alone.
    B, H, Sq, Skv, D = 1, 2, 96, 40, 128
    q, k, v, go = make(12, B, H, H, Sq, Skv, D, capi.BF16)
    out, dq, dk, dv = host.sdpa_backward(q, k, v, go, capi.BF16, causal=True)
    dead = Sq - Skv
    assert np.isnan(out[:, :, :dead]).all() and not np.isnan(out[:, :, dead:]).any()
    assert not dq[:, :, :dead].any()
    rq, rk, rv = BW.sdpa_backward(q[:, :, dead:], k, v, go[:, :, dead:], causal=True)
    compare("dq (live rows)", dq[:, :, dead:], rq)
    compare("dk", dk, rk)
    compare("dv", dv, rv)
    # a sequence with no keys at all: zero gradients everywhere for it
    lens = np.array([0], np.int32)
    out, dq, dk, dv = host.sdpa_backward(q[:, :, :40], k, v, go[:, :, :40], capi.BF16, kv_lens=lens)
    assert not dq.any() and not dk.any() and not dv.any()


@pytest.mark.parametrize("D", [128, 64])
def test_backward_at_a_few_thousand_tokens(gpu, D):
    B, Hq, Hkv, S = 1, 4, 2, 2048
    q, k, v, go = make(13, B, Hq, Hkv, S, S, D, capi.BF16)
    out, dq, dk, dv = host.sdpa_backward(q, k, v, go, capi.BF16, causal=True)
    rq, rk, rv = BW.sdpa_backward(q.reshape(B, Hkv, 2, S, D), k[:, :, None], v[:, :, None], go.reshape(B, Hkv, 2, S, D), causal=True)
    compare("dq", dq, rq.reshape(B, Hq, S, D))
    compare("dk", dk, rk.reshape(B, Hkv, S, D))
    compare("dv", dv, rv.reshape(B, Hkv, S, D))


def make_d(seed, B, Hq, Hkv, Sq, Skv, D, Dv, dtype):
    r = np.random.Generator(np.random.PCG64(seed))
    mk = lambda *s: dtypes.round_to(r.standard_normal(s, dtype=np.float32), dtype)
    return mk(B, Hq, Sq, D), mk(B, Hkv, Skv, D), mk(B, Hkv, Skv, Dv), mk(B, Hq, Sq, Dv)


@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, D, Dv, causal, kv_lens, mask kind
    (2, 2, 2, 4, 4, 8, 8, False, None, None),                    # the reference's smoke shape (shape_ops.rs:1575-1591)
    (1, 3, 3, 33, 65, 16, 24, False, None, None),                # D != Dv, lengths off the 32-wide tiles
    (2, 4, 2, 70, 70, 64, 64, True, None, None),
    (2, 4, 1, 50, 90, 40, 40, True, [90, 37], None),             # grouped queries, causal alignment, ragged keys
    (2, 2, 2, 45, 61, 32, 32, False, None, "full"),              # dense additive mask with -inf holes
    (2, 3, 3, 40, 40, 128, 128, False, None, "row"),             # [1, 1, 1, Skv] mask: broadcast over batch, head, row
    (1, 2, 2, 20, 30, 256, 200, True, None, "head"),             # the widest heads, [1, H, Sq, Skv] mask on top of causal
], ids=["ref_smoke", "d_ne_dv", "causal", "gqa_ragged", "mask_full", "mask_row", "wide_mask_head"])
def test_generic_backward_f32_against_the_oracle(gpu, shape):
    """The reference's own dtype through the generic kernels: 1e-5 of the largest gradient magnitude against the f64 oracle
    (f32 products and sums in a different order than the reference's tape; measured about 1e-6)."""
    B, Hq, Hkv, Sq, Skv, D, Dv, causal, lens, mk = shape
    G = Hq // Hkv
    say("generic backward f32: %s" % (shape,))
    q, k, v, go = make_d(21, B, Hq, Hkv, Sq, Skv, D, Dv, capi.F32)
    r = np.random.Generator(np.random.PCG64(22))
    mask = None
    if mk is not None:
        mshape = {"full": (B, Hq, Sq, Skv), "row": (1, 1, 1, Skv), "head": (1, Hq, Sq, Skv)}[mk]
        mask = r.standard_normal(mshape, dtype=np.float32)
        mask[r.random(mshape) < 0.25] = -np.inf
        mask[..., 0] = 0.0                                       # every row keeps a visible key
    lens_a = None if lens is None else np.asarray(lens, np.int32)
    out, dq, dk, dv = host.sdpa_backward(q, k, v, go, capi.F32, causal=causal, kv_lens=lens_a, mask=mask, impl=capi.IMPL_GENERIC)
    m5 = None if mask is None else np.broadcast_to(mask, (B, Hq, Sq, Skv)).reshape(B, Hkv, G, Sq, Skv)
    rq, rk, rv = BW.sdpa_backward(q.reshape(B, Hkv, G, Sq, D), k[:, :, None], v[:, :, None], go.reshape(B, Hkv, G, Sq, Dv),
                                  mask=m5, causal=causal, kv_lens=None if lens is None else lens_a.reshape(B, 1, 1))
    compare("dq", dq, rq.reshape(B, Hq, Sq, D), tol=1e-5)
    compare("dk", dk, rk.reshape(B, Hkv, Skv, D), tol=1e-5)
    compare("dv", dv, rv.reshape(B, Hkv, Skv, Dv), tol=1e-5)


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16, capi.F32], ids=lambda x: dtypes.NAMES[x])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, D, Dv, causal, kv_lens, mask kind
    (2, 2, 2, 150, 200, 128, 128, False, None, "full"),            # values with -inf holes, a mask of its own per batch entry and head
    (2, 4, 2, 130, 130, 64, 64, True, None, "head"),               # grouped queries: [1, Hq, Sq, Skv] on top of the causal flag
    (2, 3, 3, 100, 260, 128, 128, False, [260, 90], "row"),        # [1, 1, 1, Skv]: one row for everybody, with key counts
    (1, 2, 2, 200, 200, 96, 72, False, None, "causal_tensor"),     # the causal mask as a tensor (no flag), padded head dimensions
    (2, 2, 1, 70, 333, 128, 128, False, None, "batch"),            # [B, 1, Sq, Skv]; 333 keys: rows of the mask are not 8-byte aligned
    (1, 4, 2, 330, 400, 128, 128, False, None, "causal_bias"),     # per-head distance bias under the causal triangle: blocks of all kinds
    (2, 2, 2, 300, 304, 64, 64, False, None, "window"),            # a band of 70 keys: hidden blocks on both sides, zeros between
    (1, 2, 1, 257, 296, 128, 128, True, None, "blocks"),           # random 32 x 32 blocks hidden / zero / values, under the causal flag
], ids=["full", "gqa_head_causal", "row_lens", "causal_tensor", "batch_unaligned", "causal_bias", "window", "blocks"])
def test_matrix_core_backward_with_a_dense_mask(gpu, dtype, shape):
    """Gradients with a dense additive mask run on the matrix-core kernels, 16-bit and f32 (instances that add the mask's values
    to the scores before the exponential): against the f64 oracle, AUTO picks them, and the generic kernels agree."""
    B, Hq, Hkv, Sq, Skv, D, Dv, causal, lens, mk = shape
    G = Hq // Hkv
    say("matrix-core backward with a mask: %s %s" % (dtypes.NAMES[dtype], shape))
    q, k, v, go = make_d(71 + Sq, B, Hq, Hkv, Sq, Skv, D, Dv, dtype)
    r = np.random.Generator(np.random.PCG64(72))
    if mk == "causal_tensor":
        mask = np.triu(np.full((Sq, Skv), -np.inf, np.float32), 1 + Skv - Sq).reshape(1, 1, Sq, Skv)
    elif mk == "causal_bias":
        dist = (np.arange(Sq)[:, None] + (Skv - Sq) - np.arange(Skv)[None, :]).astype(np.float32)
        mask = np.where(dist >= 0, -dist[None] * (0.5 ** np.arange(1, Hq + 1, dtype=np.float32))[:, None, None], -np.inf)[None].astype(np.float32)
    elif mk == "window":
        dist = np.arange(Sq)[:, None] + (Skv - Sq) - np.arange(Skv)[None, :]
        mask = np.where((dist >= 0) & (dist < 70), 0.0, -np.inf).astype(np.float32).reshape(1, 1, Sq, Skv)
    elif mk == "blocks":
        kinds = r.integers(0, 3, size=(B, Hq, (Sq + 31) // 32, (Skv + 31) // 32))
        kinds[..., 0] = 1                                        # every row keeps visible keys
        big = np.repeat(np.repeat(kinds, 32, axis=2), 32, axis=3)[:, :, :Sq, :Skv]
        mask = np.where(big == 0, -np.inf, np.where(big == 1, 0.0, r.standard_normal((B, Hq, Sq, Skv), dtype=np.float32))).astype(np.float32)
    else:
        mshape = {"full": (B, Hq, Sq, Skv), "row": (1, 1, 1, Skv), "head": (1, Hq, Sq, Skv), "batch": (B, 1, Sq, Skv)}[mk]
        mask = r.standard_normal(mshape, dtype=np.float32)
        mask[r.random(mshape) < 0.25] = -np.inf
        mask[..., 0] = 0.0                                       # every row keeps a visible key
    mask = dtypes.round_to(mask, dtype)
    lens_a = None if lens is None else np.asarray(lens, np.int32)
    kw = dict(causal=causal, kv_lens=lens_a, mask=mask)
    out, dq, dk, dv = host.sdpa_backward(q, k, v, go, dtype, impl=capi.IMPL_MFMA, **kw)
    auto = host.sdpa_backward(q, k, v, go, dtype, **kw)
    gen = host.sdpa_backward(q, k, v, go, dtype, impl=capi.IMPL_GENERIC, **kw)
    m5 = np.broadcast_to(mask, (B, Hq, Sq, Skv)).reshape(B, Hkv, G, Sq, Skv)
    rq, rk, rv = BW.sdpa_backward(q.reshape(B, Hkv, G, Sq, D), k[:, :, None], v[:, :, None], go.reshape(B, Hkv, G, Sq, Dv),
                                  mask=m5, causal=causal, kv_lens=None if lens is None else lens_a.reshape(B, 1, 1))
    f32 = dtype == capi.F32
    for name, x, a, gx, r_ in zip(("dq", "dk", "dv"), (dq, dk, dv), auto[1:], gen[1:],
                                  (rq.reshape(B, Hq, Sq, D), rk.reshape(B, Hkv, Skv, D), rv.reshape(B, Hkv, Skv, Dv))):
        compare(name, x, r_, tol=1e-5 if f32 else 2e-2)
        if f32:       # (AUTO's forward of an f32 launch this small may be another kernel: last-bit differences in O and lse)
            compare(name + " AUTO vs pinned", a, x, tol=2e-6)
        else:
            assert np.array_equal(x, a), name + ": AUTO takes the same kernels"
        compare(name + " generic vs matrix-core", gx, x, tol=1e-5 if f32 else 1e-2)


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16, capi.F32], ids=lambda x: dtypes.NAMES[x])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, D, causal, mask kind
    (1, 4, 2, 1100, 1400, 128, True, "blocks"),
    (1, 2, 2, 1300, 1304, 64, False, "band"),
    (2, 2, 1, 900, 1600, 128, False, "values"),
    (1, 2, 2, 1027, 1501, 64, True, "blocks"),          # rows of the mask that cannot be copied 16 bytes at a time
], ids=["blocks_gqa128", "band64", "values128", "blocks_unaligned64"])
def test_matrix_core_backward_with_a_dense_mask_over_many_tiles(gpu, dtype, shape):
    """Masks over 14 - 25 tiles of keys and of query rows, where the kernels' look-ahead (flags two tiles ahead, values or their
    copies into LDS one ahead, tile ranges trimmed by the flags) runs at length: random blocks of 32 x 32 that are hidden, zero or
    valued (runs of each), a band of values around the diagonal with -inf away from it, values with holes everywhere."""
    B, Hq, Hkv, Sq, Skv, D, causal, mk = shape
    G = Hq // Hkv
    say("matrix-core backward with a mask over many tiles: %s %s" % (dtypes.NAMES[dtype], shape))
    q, k, v, go = make(81 + Sq, B, Hq, Hkv, Sq, Skv, D, dtype)
    r = np.random.Generator(np.random.PCG64(82))
    if mk == "blocks":
        kinds = r.integers(0, 3, size=(1, Hq, (Sq + 31) // 32, (Skv + 31) // 32))
        kinds[..., 0] = 1                                        # every row keeps visible keys
        big = np.repeat(np.repeat(kinds, 32, axis=2), 32, axis=3)[:, :, :Sq, :Skv]
        mask = np.where(big == 0, -np.inf, np.where(big == 1, 0.0, r.standard_normal((1, Hq, Sq, Skv), dtype=np.float32))).astype(np.float32)
    elif mk == "band":
        dist = np.abs(np.arange(Sq)[:, None] - np.arange(Skv)[None, :])
        mask = np.where(dist > 300, -np.inf, np.where(dist < 100, r.standard_normal((Sq, Skv)), 0.0)).astype(np.float32).reshape(1, 1, Sq, Skv)
    else:
        mask = r.standard_normal((B, 1, Sq, Skv), dtype=np.float32)
        mask[r.random(mask.shape) < 0.25] = -np.inf
        mask[..., 0] = 0.0
    mask = dtypes.round_to(mask, dtype)
    out, dq, dk, dv = host.sdpa_backward(q, k, v, go, dtype, causal=causal, mask=mask)
    m5 = np.broadcast_to(mask, (B, Hq, Sq, Skv)).reshape(B, Hkv, G, Sq, Skv)
    rq, rk, rv = BW.sdpa_backward(q.reshape(B, Hkv, G, Sq, D), k[:, :, None], v[:, :, None], go.reshape(B, Hkv, G, Sq, D), mask=m5, causal=causal)
    assert not np.isnan(rq).any(), "case construction: a row without keys"
    tol = 1e-5 if dtype == capi.F32 else 2e-2
    compare("dq", dq, rq.reshape(B, Hq, Sq, D), tol=tol)
    compare("dk", dk, rk.reshape(B, Hkv, Skv, D), tol=tol)
    compare("dv", dv, rv.reshape(B, Hkv, Skv, D), tol=tol)


def test_backward_random_cases_with_a_dense_mask(gpu):
    """Seeded random shapes with a mask tensor on the matrix-core backward kernels, all three dtypes: values with holes, blocks
    of 32 x 32 hidden / zero / valued at random, a band; any leading axis of the mask broadcast; lengths on either side of the
    tiles; with and without the causal flag and key counts.  Column 0 of every mask row stays visible (and row 0 sees key 0
    under the causal alignment with Sq <= Skv), so the oracle has no NaN.  Each case is printed before it runs."""
    r = np.random.Generator(np.random.PCG64(2027))
    for case in range(30):
        dtype = (capi.BF16, capi.F16, capi.F32)[case % 3]
        D = 128 if case % 2 else 64
        B, Hkv, G = int(r.integers(1, 3)), int(r.integers(1, 3)), int(r.choice([1, 2, 4]))
        Skv = int(r.choice([r.integers(1, 70), r.integers(60, 140), r.integers(120, 420)]))
        if case % 4 < 2:
            Skv = (Skv + 7) // 8 * 8          # (rows the 16-bit dK/dV kernel can copy into LDS)
        causal = bool(r.integers(0, 2))
        Sq = int(r.integers(1, Skv + 1)) if causal else int(r.integers(1, 300))
        lens = r.integers(1, Skv + 1, B).astype(np.int32) if r.integers(0, 2) else None
        Hq = Hkv * G
        shp = [B if r.random() < 0.5 else 1, Hq if r.random() < 0.5 else 1, Sq if r.random() < 0.8 else 1, Skv]
        kind = str(r.choice(["holes", "blocks", "band"]))
        mask = r.standard_normal(shp, dtype=np.float32)
        if kind == "holes":
            mask[r.random(shp) < 0.25] = -np.inf
        elif kind == "blocks":
            kinds = r.integers(0, 3, size=(shp[0], shp[1], (shp[2] + 31) // 32, (Skv + 31) // 32))
            big = np.repeat(np.repeat(kinds, 32, axis=2), 32, axis=3)[:, :, :shp[2], :Skv]
            mask = np.where(big == 0, -np.inf, np.where(big == 1, 0.0, mask)).astype(np.float32)
        elif shp[2] > 1:
            dist = np.arange(Sq)[:, None] + (Skv - Sq) - np.arange(Skv)[None, :]
            mask = np.where((np.abs(dist) <= int(r.integers(8, 120)))[None, None], 0.1 * mask, -np.inf).astype(np.float32)
        mask[..., 0] = 0.0
        mask = dtypes.round_to(mask, dtype)
        say("masked backward random case %d: dtype=%d D=%d B=%d Hq=%d Hkv=%d Sq=%d Skv=%d causal=%s lens=%s mask %s %r"
            % (case, dtype, D, B, Hq, Hkv, Sq, Skv, causal, None if lens is None else lens.tolist(), kind, tuple(shp)))
        q, k, v, go = make(300 + case, B, Hq, Hkv, Sq, Skv, D, dtype)
        out, dq, dk, dv = host.sdpa_backward(q, k, v, go, dtype, causal=causal, kv_lens=lens, mask=mask, impl=capi.IMPL_MFMA)
        m5 = np.broadcast_to(mask, (B, Hq, Sq, Skv)).reshape(B, Hkv, G, Sq, Skv)
        rq, rk, rv = BW.sdpa_backward(q.reshape(B, Hkv, G, Sq, D), k[:, :, None], v[:, :, None], go.reshape(B, Hkv, G, Sq, D),
                                      mask=m5, causal=causal, kv_lens=None if lens is None else lens.reshape(B, 1, 1))
        assert not np.isnan(rq).any(), "case construction: a row without keys"
        tol = 1e-5 if dtype == capi.F32 else 2e-2
        compare("dq", dq, rq.reshape(B, Hq, Sq, D), tol=tol)
        compare("dk", dk, rk.reshape(B, Hkv, Skv, D), tol=tol)
        compare("dv", dv, rv.reshape(B, Hkv, Skv, D), tol=tol)


@pytest.mark.parametrize("dtype,dims", [(capi.BF16, (96, 96)), (capi.BF16, (40, 72)), (capi.F16, (128, 64)), (capi.BF16, (8, 8)), (capi.F16, (80, 80)),
                                        (capi.F32, (96, 96)), (capi.F32, (20, 36)), (capi.F32, (128, 64)), (capi.F32, (4, 4))],
                         ids=lambda x: dtypes.NAMES[x] if isinstance(x, int) else "D%d_Dv%d" % x)
def test_matrix_core_backward_with_padded_head_dimensions(gpu, dtype, dims):
    """Head dimensions up to 128 in whole 16-byte vectors, D and Dv not necessarily equal, through the matrix-core backward
    kernels (pinned, and AUTO must pick them): zero-padded into the 64 / 128 instances, gradient stores cut at D and Dv."""
    D, Dv = dims
    tol = 1e-5 if dtype == capi.F32 else 2e-2
    for B, Hq, Hkv, Sq, Skv, causal, lens in ((2, 4, 2, 150, 200, True, [200, 77]), (1, 2, 2, 70, 70, False, None)):
        G = Hq // Hkv
        say("padded backward: %s D=%d Dv=%d %r" % (dtypes.NAMES[dtype], D, Dv, (B, Hq, Hkv, Sq, Skv)))
        q, k, v, go = make_d(61 + D, B, Hq, Hkv, Sq, Skv, D, Dv, dtype)
        lens_a = None if lens is None else np.asarray(lens, np.int32)
        out, dq, dk, dv = host.sdpa_backward(q, k, v, go, dtype, causal=causal, kv_lens=lens_a, impl=capi.IMPL_MFMA)
        auto = host.sdpa_backward(q, k, v, go, dtype, causal=causal, kv_lens=lens_a)
        rq, rk, rv = BW.sdpa_backward(q.reshape(B, Hkv, G, Sq, D), k[:, :, None], v[:, :, None], go.reshape(B, Hkv, G, Sq, Dv),
                                      causal=causal, kv_lens=None if lens is None else lens_a.reshape(B, 1, 1))
        for name, x, a, r_ in zip(("dq", "dk", "dv"), (dq, dk, dv), auto[1:], (rq.reshape(B, Hq, Sq, D), rk.reshape(B, Hkv, Skv, D), rv.reshape(B, Hkv, Skv, Dv))):
            compare(name, x, r_, tol=tol)
            if dtype == capi.F32:       # (AUTO's forward of an f32 launch this small is the split-KV kernel: last-bit differences in O and lse)
                compare(name + " AUTO vs pinned", a, x, tol=2e-6)
            else:
                assert np.array_equal(x, a), name + ": AUTO takes the same kernels"


@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, D, causal, kv_lens, scale
    (1, 1, 1, 32, 32, 64, False, None, None),
    (1, 1, 1, 32, 32, 128, True, None, None),
    (2, 3, 3, 128, 128, 64, True, None, None),                   # the reference's bench head shape, causal
    (2, 4, 4, 200, 333, 64, False, None, 0.3),
    (2, 4, 2, 300, 300, 128, True, None, None),
    (1, 8, 2, 130, 450, 64, True, None, None),                   # Sq < Skv: causal alignment, grouped queries
    (3, 2, 2, 257, 257, 64, True, [257, 100, 31], None),
    (2, 2, 1, 64, 700, 128, False, [700, 2], None),
    (1, 2, 2, 513, 129, 64, False, None, -0.125),                # a negative scale is a scale like any other in f32
    (8, 2, 1, 77, 140, 128, True, [140, 70, 64, 65, 128, 129, 100, 96], None),      # (batch, KV head) pairs dealt over the XCDs
], ids=["tiny64", "tiny128_causal", "bench_head", "rect", "gqa_causal128", "gqa_rect_causal", "ragged_causal", "ragged128",
        "negative_scale", "dealt_pairs"])
def test_matrix_core_backward_f32_against_the_oracle(gpu, shape):
    """f32 through the IEEE-f32 matrix-core kernels (D = 64 and 128), picked by AUTO and pinned: 1e-5 of the largest
    gradient magnitude against the f64 oracle, and the generic f32 kernels within the same distance."""
    B, Hq, Hkv, Sq, Skv, D, causal, lens, scale = shape
    G = Hq // Hkv
    say("matrix-core backward f32: %s" % (shape,))
    q, k, v, go = make(41, B, Hq, Hkv, Sq, Skv, D, capi.F32)
    lens_a = None if lens is None else np.asarray(lens, np.int32)
    kw = dict(causal=causal, kv_lens=lens_a, scale=scale)
    out, dq, dk, dv = host.sdpa_backward(q, k, v, go, capi.F32, impl=capi.IMPL_MFMA, **kw)
    auto = host.sdpa_backward(q, k, v, go, capi.F32, **kw)
    gen = host.sdpa_backward(q, k, v, go, capi.F32, impl=capi.IMPL_GENERIC, **kw)
    rq, rk, rv = BW.sdpa_backward(q.reshape(B, Hkv, G, Sq, D), k[:, :, None], v[:, :, None], go.reshape(B, Hkv, G, Sq, D),
                                  scale=scale, causal=causal, kv_lens=None if lens is None else lens_a.reshape(B, 1, 1))
    refs = (rq.reshape(B, Hq, Sq, D), rk.reshape(B, Hkv, Skv, D), rv.reshape(B, Hkv, Skv, D))
    for name, x, a, g_, r_ in zip(("dq", "dk", "dv"), (dq, dk, dv), auto[1:], gen[1:], refs):
        compare(name, x, r_, tol=1e-5)
        # (AUTO's forward of launches this small is the f32 split-KV kernel: O and the row normalisers differ in the last bits)
        compare(name + " AUTO vs pinned", a, x, tol=2e-6)
        compare(name + " generic vs matrix-core", g_, x, tol=2e-5)
    if lens is not None:
        for b in range(B):
            assert not dk[b, :, lens[b]:].any() and not dv[b, :, lens[b]:].any()      # padded keys: exactly zero


@pytest.mark.parametrize("parts", ["1", "2", "4"])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, D, Dv, causal, kv_lens, q_lens, mask
    (1, 4, 4, 1024, 1024, 64, 64, True, None, None, None),
    (2, 4, 2, 600, 1100, 128, 128, True, [1100, 300], None, None),           # a sequence whose keys end inside the first part
    (1, 2, 2, 1030, 520, 64, 32, False, None, None, None),                  # D != Dv: planes of different widths
    (1, 8, 2, 520, 1500, 128, 128, True, None, None, "window"),             # a mask whose block flags trim the walk before it is dealt
    (2, 2, 2, 1024, 1024, 64, 64, True, [1024, 700], [1024, 700], None),    # padding rows: zero in every plane
    (1, 2, 1, 300, 2100, 64, 64, False, None, None, "values"),
], ids=["causal", "ragged_gqa128", "rect_d_dv", "window_gqa128", "padded", "values"])
def test_matrix_core_backward_f32_in_parts(gpu, monkeypatch, parts, shape):
    """The f32 matrix-core kernels with the tiles of a block dealt to 1, 2 and 4 workgroups whose sums meet in planes of the
    workspace (what a call that does not fill the device gets by itself; INCIN_ROCM_BWD_PARTS forces it): 1e-5 of the largest
    gradient magnitude against the f64 oracle each, exact zeros where padding is."""
    B, Hq, Hkv, Sq, Skv, D, Dv, causal, lens, qlens, mk = shape
    G = Hq // Hkv
    monkeypatch.setenv("INCIN_ROCM_BWD_PARTS", parts)
    say("matrix-core backward f32 in %s parts: %s" % (parts, shape))
    q, k, v, go = make_d(91 + Sq, B, Hq, Hkv, Sq, Skv, D, Dv, capi.F32)
    r = np.random.Generator(np.random.PCG64(92))
    mask = None
    if mk == "window":
        dist = np.arange(Sq)[:, None] + (Skv - Sq) - np.arange(Skv)[None, :]
        mask = np.where((dist >= 0) & (dist < 400), 0.0, -np.inf).astype(np.float32).reshape(1, 1, Sq, Skv)
    elif mk == "values":
        mask = r.standard_normal((1, Hq, Sq, Skv), dtype=np.float32)
        mask[r.random(mask.shape) < 0.25] = -np.inf
        mask[..., 0] = 0.0
    lens_a = None if lens is None else np.asarray(lens, np.int32)
    qlens_a = None if qlens is None else np.asarray(qlens, np.int32)
    out, dq, dk, dv = host.sdpa_backward(q, k, v, go, capi.F32, impl=capi.IMPL_MFMA, causal=causal, kv_lens=lens_a, q_lens=qlens_a, mask=mask,
                                         poison_padding=qlens is not None)
    for b in range(B):
        nq = Sq if qlens is None else int(qlens[b])
        nk = Skv if lens is None else int(lens[b])
        m5 = None if mask is None else np.broadcast_to(mask, (B, Hq, Sq, Skv))[b:b + 1, :, :nq, :nk].reshape(1, Hkv, G, nq, nk)
        # (a sequence cut to its lengths: the causal diagonal is anchored at the full extents)
        if causal and (nq != Sq or nk != Skv) and nk - nq != Skv - Sq:
            tri = np.triu(np.full((Sq, Skv), -np.inf, np.float32), 1 + Skv - Sq)[:nq, :nk].reshape(1, 1, 1, nq, nk)
            m5 = tri if m5 is None else m5 + tri
            cz = False
        else:
            cz = causal
        rq, rk, rv = BW.sdpa_backward(q[b:b + 1, :, :nq].reshape(1, Hkv, G, nq, D), k[b:b + 1, :, None, :nk], v[b:b + 1, :, None, :nk],
                                      go[b:b + 1, :, :nq].reshape(1, Hkv, G, nq, Dv), mask=m5, causal=cz)
        compare("dq[%d]" % b, dq[b:b + 1, :, :nq], rq.reshape(1, Hq, nq, D), tol=1e-5)
        compare("dk[%d]" % b, dk[b:b + 1, :, :nk], rk.reshape(1, Hkv, nk, D), tol=1e-5)
        compare("dv[%d]" % b, dv[b:b + 1, :, :nk], rv.reshape(1, Hkv, nk, Dv), tol=1e-5)
        assert not dq[b, :, nq:].any() and not dk[b, :, nk:].any() and not dv[b, :, nk:].any()


@pytest.mark.parametrize("parts", ["1", "2", "4", "8"])
@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16], ids=lambda x: dtypes.NAMES[x])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, D, Dv, causal, kv_lens, q_lens, mask
    (1, 8, 1, 1024, 1024, 128, 128, True, None, None, None),                # eight query heads walking one KV head's key blocks
    (2, 4, 2, 600, 1100, 64, 64, True, [1100, 300], None, None),
    (1, 2, 2, 2100, 520, 128, 64, False, None, None, None),                 # D != Dv: planes of different widths
    (1, 8, 2, 520, 1504, 128, 128, True, None, None, "window"),             # a mask whose values go through LDS; its flags trim the walk before it is dealt
    (2, 2, 2, 1024, 1024, 64, 64, True, [1024, 700], [1024, 700], None),    # padding rows and keys: zero in every plane
    (1, 4, 1, 700, 333, 128, 128, False, None, None, "values"),             # a mask whose rows cannot be copied
], ids=["gqa8", "ragged_gqa64", "rect_d_dv", "window_gqa", "padded", "values_unaligned"])
def test_matrix_core_backward_16bit_in_parts(gpu, monkeypatch, parts, dtype, shape):
    """The 16-bit dK/dV kernel with the walk of a key block - the query tiles of every head of its group - dealt to 1, 2, 4 and 8
    workgroups whose sums meet as f32 in planes of the workspace (what a call with few key blocks gets by itself;
    INCIN_ROCM_BWD_PARTS forces it): against the f64 oracle each, exact zeros where padding is."""
    B, Hq, Hkv, Sq, Skv, D, Dv, causal, lens, qlens, mk = shape
    G = Hq // Hkv
    monkeypatch.setenv("INCIN_ROCM_BWD_PARTS", parts)
    say("matrix-core backward %s in %s parts: %s" % (dtypes.NAMES[dtype], parts, shape))
    q, k, v, go = make_d(95 + Sq, B, Hq, Hkv, Sq, Skv, D, Dv, dtype)
    r = np.random.Generator(np.random.PCG64(96))
    mask = None
    if mk == "window":
        dist = np.arange(Sq)[:, None] + (Skv - Sq) - np.arange(Skv)[None, :]
        mask = np.where((dist >= 0) & (dist < 400), -0.01 * dist, -np.inf).astype(np.float32).reshape(1, 1, Sq, Skv)
    elif mk == "values":
        mask = r.standard_normal((1, Hq, Sq, Skv), dtype=np.float32)
        mask[r.random(mask.shape) < 0.25] = -np.inf
        mask[..., 0] = 0.0
    if mask is not None:
        mask = dtypes.round_to(mask, dtype)
    lens_a = None if lens is None else np.asarray(lens, np.int32)
    qlens_a = None if qlens is None else np.asarray(qlens, np.int32)
    out, dq, dk, dv = host.sdpa_backward(q, k, v, go, dtype, impl=capi.IMPL_MFMA, causal=causal, kv_lens=lens_a, q_lens=qlens_a, mask=mask,
                                         poison_padding=qlens is not None)
    for b in range(B):
        nq = Sq if qlens is None else int(qlens[b])
        nk = Skv if lens is None else int(lens[b])
        m5 = None if mask is None else np.broadcast_to(mask, (B, Hq, Sq, Skv))[b:b + 1, :, :nq, :nk].reshape(1, Hkv, G, nq, nk)
        if causal and nk - nq != Skv - Sq:      # (a sequence cut to its lengths: the causal diagonal stays anchored at the full extents)
            tri = np.triu(np.full((Sq, Skv), -np.inf, np.float32), 1 + Skv - Sq)[:nq, :nk].reshape(1, 1, 1, nq, nk)
            m5 = tri if m5 is None else m5 + tri
            cz = False
        else:
            cz = causal
        rq, rk, rv = BW.sdpa_backward(q[b:b + 1, :, :nq].reshape(1, Hkv, G, nq, D), k[b:b + 1, :, None, :nk], v[b:b + 1, :, None, :nk],
                                      go[b:b + 1, :, :nq].reshape(1, Hkv, G, nq, Dv), mask=m5, causal=cz)
        compare("dq[%d]" % b, dq[b:b + 1, :, :nq], rq.reshape(1, Hq, nq, D))
        compare("dk[%d]" % b, dk[b:b + 1, :, :nk], rk.reshape(1, Hkv, nk, D))
        compare("dv[%d]" % b, dv[b:b + 1, :, :nk], rv.reshape(1, Hkv, nk, Dv))
        assert not dq[b, :, nq:].any() and not dk[b, :, nk:].any() and not dv[b, :, nk:].any()


def test_matrix_core_backward_f32_rows_without_keys(gpu):
    # Sq > Skv under causal alignment: the first Sq - Skv rows see nothing; they get a zero dq and add nothing to dk, dv
    B, H, Sq, Skv, D = 1, 2, 96, 40, 64
    q, k, v, go = make(42, B, H, H, Sq, Skv, D, capi.F32)
    out, dq, dk, dv = host.sdpa_backward(q, k, v, go, capi.F32, causal=True, impl=capi.IMPL_MFMA)
    dead = Sq - Skv
    assert np.isnan(out[:, :, :dead]).all() and not dq[:, :, :dead].any()
    rq, rk, rv = BW.sdpa_backward(q[:, :, dead:], k, v, go[:, :, dead:], causal=True)
    compare("dq (live rows)", dq[:, :, dead:], rq, tol=1e-5)
    compare("dk", dk, rk, tol=1e-5)
    compare("dv", dv, rv, tol=1e-5)
    lens = np.array([0], np.int32)
    out, dq, dk, dv = host.sdpa_backward(q[:, :, :40], k, v, go[:, :, :40], capi.F32, kv_lens=lens, impl=capi.IMPL_MFMA)
    assert not dq.any() and not dk.any() and not dv.any()


def test_matrix_core_backward_f32_single_key(gpu):
    """One visible key: P = 1, dS = dP - D = 0 and dq = dk = 0 in real arithmetic.  The reference's tape subtracts dP from
    itself there (cpu/ops/elementwise.rs:1062-1077: the sum over one element) and gets an exact zero; the kernels subtract
    D_i = dO_i . O_i from dP_i0 = dO_i . V_0, two f32 evaluations of one sum of D products, each off by the rounding of its
    partial sums (of the order of sqrt(D) half units in the last place).  What reaches the gradients is bounded by that:
    2 sqrt(D) 2^-24 max|dP| per dS, times |scale| sum_i |Q_id| for dk and |scale| |K_0d| for dq; dv is the plain column sum
    of dO."""
    B, Hq, Hkv, Sq, Skv, D = 1, 2, 1, 64, 70, 128
    q, k, v, go = make(44, B, Hq, Hkv, Sq, Skv, D, capi.F32)
    lens = np.array([1], np.int32)
    out, dq, dk, dv = host.sdpa_backward(q, k, v, go, capi.F32, kv_lens=lens, impl=capi.IMPL_MFMA)
    s = 1.0 / np.sqrt(D)
    eps_ds = 2.0 * np.sqrt(D) * 2.0 ** -24 * float(np.abs(go.astype(np.float64) @ v[0, 0, 0].astype(np.float64)).max())
    say("   single key: max|dq| %.3e max|dk| %.3e, dS rounding level %.3e" % (np.abs(dq).max(), np.abs(dk).max(), eps_ds))
    assert np.abs(dq).max() <= eps_ds * s * np.abs(k[0, 0, 0]).max()
    assert np.abs(dk[0, 0, 0]).max() <= eps_ds * s * np.abs(q).sum(axis=(1, 2)).max()
    assert not dk[0, 0, 1:].any() and not dv[0, 0, 1:].any()
    compare("dv", dv[0, 0, 0], go.astype(np.float64).sum(axis=(0, 1, 2)), tol=1e-5)


def test_matrix_core_backward_f32_at_a_few_thousand_tokens(gpu):
    B, Hq, Hkv, S, D = 1, 4, 2, 2048, 128
    q, k, v, go = make(43, B, Hq, Hkv, S, S, D, capi.F32)
    out, dq, dk, dv = host.sdpa_backward(q, k, v, go, capi.F32, causal=True, impl=capi.IMPL_MFMA)
    rq, rk, rv = BW.sdpa_backward(q.reshape(B, Hkv, 2, S, D), k[:, :, None], v[:, :, None], go.reshape(B, Hkv, 2, S, D), causal=True)
    compare("dq", dq, rq.reshape(B, Hq, S, D), tol=1e-5)
    compare("dk", dk, rk.reshape(B, Hkv, S, D), tol=1e-5)
    compare("dv", dv, rv.reshape(B, Hkv, S, D), tol=1e-5)


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16])
@pytest.mark.parametrize("D", [128, 64])
def test_generic_and_matrix_core_backward_agree(gpu, dtype, D):
    """The same 16-bit problem through both sets of kernels: each within tolerance of the oracle, and of each other."""
    B, Hq, Hkv, S = 2, 4, 2, 200
    q, k, v, go = make(31, B, Hq, Hkv, S, S, D, dtype)
    lens = np.array([200, 77], np.int32)
    a = host.sdpa_backward(q, k, v, go, dtype, causal=True, kv_lens=lens, impl=capi.IMPL_GENERIC)
    b = host.sdpa_backward(q, k, v, go, dtype, causal=True, kv_lens=lens, impl=capi.IMPL_MFMA)
    ref = BW.sdpa_backward(q.reshape(B, Hkv, 2, S, D), k[:, :, None], v[:, :, None], go.reshape(B, Hkv, 2, S, D),
                           causal=True, kv_lens=lens.reshape(B, 1, 1))
    shapes = [(B, Hq, S, D), (B, Hkv, S, D), (B, Hkv, S, D)]
    for name, x, y, r_, shp in zip(("dq", "dk", "dv"), a[1:], b[1:], ref, shapes):
        compare(name + " generic", x, r_.reshape(shp))
        compare(name + " mfma", y, r_.reshape(shp))
        compare(name + " generic vs mfma", x, y)


def test_backward_refuses_what_it_does_not_cover(gpu):
    q, k, v, go = make(14, 1, 1, 1, 32, 32, 36, capi.BF16)
    with pytest.raises(capi.RocmError) as e:                     # the matrix-core kernels, pinned, outside their domain (72-byte rows)
        host.sdpa_backward(q, k, v, go, capi.BF16, impl=capi.IMPL_MFMA)
    assert e.value.code == capi.EUNSUPPORTED
    q, k, v, go = make(14, 1, 1, 1, 8, 8, 320, capi.F32)         # wider than any kernel
    with pytest.raises(capi.RocmError) as e:
        host.sdpa_backward(q, k, v, go, capi.F32)
    assert e.value.code == capi.EUNSUPPORTED


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F32])
def test_no_keys_gives_a_zero_query_gradient(gpu, dtype):
    """Queries but no keys: the output is zeros whatever q holds, so dq is zeros (the reference's tape gives zeros), and
    the entry point promises to overwrite it; dk and dv have no elements."""
    say("backward with an empty key axis, dtype %d" % dtype)
    B, H, Sq, D = 2, 3, 50, 128
    q, _, _, go = make(5, B, H, H, Sq, 1, D, dtype)
    empty = np.zeros((B, H, 0, D), np.float32)
    tq, tg = host.DeviceTensor.from_f32(q, dtype), host.DeviceTensor.from_f32(go, dtype)
    tk, tv, tdk, tdv = (host.DeviceTensor.from_f32(empty, dtype) for _ in range(4))
    to, tdq = host.DeviceTensor((B, H, Sq, D), dtype), host.DeviceTensor((B, H, Sq, D), dtype)
    capi.check(capi.load().incin_rocm_memset(0, tdq.ptr, 0x7f, tdq.buf.nbytes))          # what an allocator may leave behind
    lse = capi.DeviceBuffer(B * H * Sq * 4)
    bd = capi.SdpaBwdDesc()
    bd.fwd = host.make_desc(tq, tk, tv, to, lse=lse)
    for name, t in (("d_o", tg), ("d_q", tdq), ("d_k", tdk), ("d_v", tdv)):
        setattr(bd, name, t.ptr)
        for i, s in enumerate(host._strides3(t.shape)):
            getattr(bd, name + "_stride")[i] = s
    assert capi.sdpa_bwd_workspace(bd) == 0
    capi.sdpa_fwd(bd.fwd)
    capi.sdpa_bwd(bd)
    capi.sync()
    assert not to.to_f32().any() and not tdq.to_f32().any()


@pytest.mark.parametrize("case", [
    # dtype, impl, D
    (capi.BF16, capi.IMPL_AUTO, 128), (capi.F16, capi.IMPL_MFMA, 64), (capi.F32, capi.IMPL_AUTO, 64), (capi.F32, capi.IMPL_MFMA, 128),
    (capi.F32, capi.IMPL_GENERIC, 80), (capi.BF16, capi.IMPL_GENERIC, 128),
], ids=["bf16_auto", "f16_mfma_d64", "f32_auto_d64", "f32_mfma", "f32_generic_d80", "bf16_generic"])
def test_backward_of_a_padded_batch(gpu, case):
    """A padded self-attention batch: sequence b has lens[b] real positions, the rest of its rows and keys are padding
    (q_lens = kv_lens = lens).  The forward leaves the padding rows of O and lse unspecified - here they are overwritten
    with NaN, and the padding rows of dO hold NaN too - and the backward must give, per sequence, the gradients of that
    sequence alone: dQ, dK, dV of the truncated problem inside the lengths, exact zeros outside."""
    dtype, impl, D = case
    B, Hq, Hkv, S = 3, 4, 2, 300
    G = Hq // Hkv
    lens = np.array([300, 131, 64], np.int32)
    q, k, v, go = make(71, B, Hq, Hkv, S, S, D, dtype)
    for b in range(B):
        go[b, :, lens[b]:] = np.nan
    out, dq, dk, dv = host.sdpa_backward(q, k, v, go, dtype, causal=True, kv_lens=lens, q_lens=lens, impl=impl, poison_padding=True)
    tol = 1e-5 if dtype == capi.F32 else 2e-2
    for b in range(B):
        n = int(lens[b])
        rq, rk, rv = BW.sdpa_backward(q[b:b + 1, :, :n].reshape(1, Hkv, G, n, D), k[b:b + 1, :, None, :n], v[b:b + 1, :, None, :n],
                                      go[b:b + 1, :, :n].reshape(1, Hkv, G, n, D), causal=True)
        compare("dq[%d]" % b, dq[b:b + 1, :, :n], rq.reshape(1, Hq, n, D), tol)
        compare("dk[%d]" % b, dk[b:b + 1, :, :n], rk.reshape(1, Hkv, n, D), tol)
        compare("dv[%d]" % b, dv[b:b + 1, :, :n], rv.reshape(1, Hkv, n, D), tol)
        assert not dq[b, :, n:].any() and not dk[b, :, n:].any() and not dv[b, :, n:].any()
