"""Parity at the full benchmark sizes (configurations 2-5).  A full CPU run of these shapes takes minutes
to hours, so each case checks (a) sampled output rows against the CPU oracle - chosen to cover the first
and last rows, rows either side of every tile / workgroup boundary and random ones - and (b) properties
that hold for every row and need no oracle: rows of softmax weights sum to one (V = 1 gives O = 1),
causality (changing keys and values a query may not see leaves its output bit-identical), split
invariance (decode: the result does not depend on the number of KV splits beyond rounding)."""
import sys

import numpy as np
import pytest

from incin_amd import capi, dtypes, host
from oracle import oracle as O

pytestmark = pytest.mark.gpu
TOL = {capi.F32: 1e-5, capi.F16: 2e-2, capi.BF16: 2e-2}


def say(msg):
    print(msg, file=sys.stderr, flush=True)


def gen(seed, shape, dtype):
    r = np.random.Generator(np.random.PCG64(seed))
    return dtypes.round_to(r.standard_normal(shape, dtype=np.float32), dtype)


def interesting_rows(r, n_flat, Sq, extra, n_random):
    """(flat batch*head index, query row) pairs: fixed rows of interest in a few heads plus random ones."""
    rows = []
    for bh in sorted(set([0, n_flat - 1, int(r.integers(0, n_flat))])):
        rows += [(bh, i) for i in extra if 0 <= i < Sq]
    rows += list(zip(r.integers(0, n_flat, n_random).tolist(), r.integers(0, Sq, n_random).tolist()))
    return np.asarray(rows, dtype=np.int64)


def check_rows(got_rows, ref_rows, tol, what):
    err = float(np.abs(got_rows - ref_rows).max())
    say("%s: %d sampled rows, max-abs err %.3e (tol %.0e)" % (what, len(got_rows), err, tol))
    assert not np.isnan(got_rows).any(), what
    assert err <= tol, "%s: %.3e > %.0e" % (what, err, tol)


def test_config2_f32_causal_full(gpu):
    B, H, S, D = 4, 8, 1024, 64
    say("config 2: f32 causal B=4 H=8 S=1024 D=64, every row against the oracle")
    q, k, v = (gen(20 + i, (B, H, S, D), capi.F32) for i in range(3))
    got = host.sdpa(q, k, v, capi.F32, causal=True)
    ref = O.sdpa(q, k, v, causal=True)
    err = float(np.abs(got - ref).max())
    say("config 2: max-abs err %.3e" % err)
    assert err <= TOL[capi.F32]


def test_config3_bf16_causal_prefill_full(gpu):
    B, H, S, D = 8, 16, 4096, 128
    dt = capi.BF16
    say("config 3: bf16 causal prefill B=8 H=16 S=4096 D=128")
    q, k, v = (gen(30 + i, (B, H, S, D), dt) for i in range(3))
    got, info = host.sdpa(q, k, v, dt, causal=True, return_info=True)
    assert info["impl"] == capi.IMPL_MFMA
    r = np.random.Generator(np.random.PCG64(33))
    extra = [0, 1, 31, 32, 63, 64, 65, 127, 128, 129, 255, 256, 2047, 2048, 4030, 4031, 4032, 4064, 4094, 4095]
    rows = interesting_rows(r, B * H, S, extra, 160)
    ref = O.sdpa_rows(q, k, v, rows, causal=True)
    check_rows(got.reshape(B * H, S, D)[rows[:, 0], rows[:, 1]], ref, TOL[dt], "config 3")
    assert not np.isnan(got).any()
    # causality: new keys / values from position 2048 on must leave rows 0..2047 bit-identical
    say("config 3: causality property")
    k2, v2 = k.copy(), v.copy()
    k2[:, :, 2048:] = gen(34, (B, H, S - 2048, D), dt)
    v2[:, :, 2048:] = gen(35, (B, H, S - 2048, D), dt)
    got2 = host.sdpa(q, k2, v2, dt, causal=True)
    assert np.array_equal(got[:, :, :2048], got2[:, :, :2048])
    assert not np.array_equal(got[:, :, 2048:], got2[:, :, 2048:])
    # weights sum to one: V = 1 gives O = 1 in every row (to one bf16 rounding of the quotient)
    say("config 3: normalisation property")
    ones = np.ones_like(v)
    got1 = host.sdpa(q, k, ones, dt, causal=True)
    assert float(np.abs(got1 - 1.0).max()) <= 2.0 ** -7


def test_config4_bf16_decode_full(gpu):
    B, H, KV, D = 32, 32, 8192, 128
    dt = capi.BF16
    say("config 4: bf16 decode B=32 H=32 KV=8192 D=128, every row against the oracle")
    q = gen(40, (B, H, 1, D), dt)
    k, v = gen(41, (B, H, KV, D), dt), gen(42, (B, H, KV, D), dt)
    got, info = host.sdpa(q, k, v, dt, return_info=True)
    assert info["impl"] == capi.IMPL_SPLITKV_MFMA and info["splits"] >= 1      # a long cache: the matrix-core split-KV kernel
    ref = O.sdpa(q, k, v)
    err = float(np.abs(got - ref).max())
    say("config 4: splits %d, max-abs err %.3e" % (info["splits"], err))
    assert err <= TOL[dt]
    # split invariance: other split counts agree with the chosen one to rounding of the bf16 output
    # and so does the vector-ALU split-KV kernel, which also stands against the oracle on its own
    for impl in (capi.IMPL_SPLITKV_MFMA, capi.IMPL_SPLITKV):
        for ns in (0, 1, 4, 16):
            other, oi = host.sdpa(q, k, v, dt, num_splits=ns, impl=impl, return_info=True)
            assert oi["impl"] == impl
            d = float(np.abs(other - got).max())
            say("config 4: kernel %d, %d splits vs %d: max-abs diff %.3e" % (impl, oi["splits"], info["splits"], d))
            assert d <= 2.0 ** -8
            if impl == capi.IMPL_SPLITKV and ns == 0:
                assert float(np.abs(other - ref).max()) <= TOL[dt]


def test_config5_gqa_ragged_causal_full(gpu):
    B, Hq, Hkv, S, D = 4, 32, 8, 16384, 128
    G = Hq // Hkv
    dt = capi.BF16
    r = np.random.Generator(np.random.PCG64(50))
    lens = r.integers(2048, 16385, B).astype(np.int32)           # drawn uniform in [2048, 16384], as the configuration says
    say("config 5: GQA bf16 causal prefill, ragged lengths %s padded to %d" % (lens.tolist(), S))
    q = gen(51, (B, Hq, S, D), dt)
    k, v = gen(52, (B, Hkv, S, D), dt), gen(53, (B, Hkv, S, D), dt)
    got, info = host.sdpa(q, k, v, dt, causal=True, kv_lens=lens, return_info=True)
    assert info["impl"] == capi.IMPL_MFMA              # what AUTO picks at every length
    # the 128-row form of the kernel on the same inputs (AUTO takes 256-row workgroups here): the same bits
    import os
    os.environ["INCIN_ROCM_PREFILL_BLOCK_ROWS"] = "128"
    try:
        got128 = host.sdpa(q, k, v, dt, causal=True, kv_lens=lens, impl=capi.IMPL_MFMA)
    finally:
        del os.environ["INCIN_ROCM_PREFILL_BLOCK_ROWS"]
    for b in range(B):
        n = int(lens[b])
        assert np.array_equal(got[b, :, :n], got128[b, :, :n]), "config 5: batch %d, 128-row vs 256-row workgroups" % b
    # sampled rows inside each sequence's valid length (rows past it are padding queries); the oracle takes
    # the reference's layout for grouped queries: q [B,Hkv,G,S,D] against k, v [B,Hkv,1,S,D]
    rows = []
    for b in range(B):
        n = int(lens[b])
        cand = [0, 1, 63, 64, 127, 128, 2047, n // 2, n - 130, n - 129, n - 65, n - 64, n - 2, n - 1]
        for hq in sorted(set([0, Hq - 1, int(r.integers(0, Hq))])):
            rows += [(b * Hq + hq, i) for i in cand if 0 <= i < n]
        rows += [(b * Hq + int(r.integers(0, Hq)), int(r.integers(0, n))) for _ in range(24)]
    rows = np.asarray(rows, dtype=np.int64)
    ref = O.sdpa_rows(q.reshape(B, Hkv, G, S, D), k[:, :, None], v[:, :, None], rows, causal=True,
                      kv_lens=lens.reshape(B, 1, 1))
    check_rows(got.reshape(B * Hq, S, D)[rows[:, 0], rows[:, 1]], ref, TOL[dt], "config 5")
    # declaring the padding rows (q_lens) leaves every valid row bit-identical; what it saves is in the bench
    say("config 5: padded-query property")
    got_q = host.sdpa(q, k, v, dt, causal=True, kv_lens=lens, q_lens=lens)
    for b in range(B):
        n = int(lens[b])
        assert np.array_equal(got[b, :, :n], got_q[b, :, :n])
    # padding keys carry weight exactly 0 in a valid row: other (finite) contents behind each length change
    # nothing there
    say("config 5: key-padding property")
    k2, v2 = k.copy(), v.copy()
    for b in range(B):
        k2[b, :, lens[b]:] *= -3.0
        v2[b, :, lens[b]:] = 1000.0
    got2 = host.sdpa(q, k2, v2, dt, causal=True, kv_lens=lens)
    for b in range(B):
        n = int(lens[b])
        assert np.array_equal(got[b, :, :n], got2[b, :, :n])
        assert not np.isnan(got2[b, :, :n]).any()


def test_config3_backward_full(gpu):
    """The backward at configuration 3's full size (bf16 causal, B=8 H=16 S=4096 D=128): two (batch, head) slices against
    the float64 backward oracle, and properties that hold for every head and need no oracle - the weights of a row sum to
    one, so sum_j dV_j = sum_i dO_i; the last key is seen by the last query only, so its dV is P_last,last * dO_last."""
    from oracle import sdpa_backward as BW
    B, H, S, D = 8, 16, 4096, 128
    say("config 3 backward at full size")
    q, k, v, go = (gen(70 + i, (B, H, S, D), capi.BF16) for i in range(4))
    out, dq, dk, dv = host.sdpa_backward(q, k, v, go, capi.BF16, causal=True)
    assert not np.isnan(dq).any() and not np.isnan(dk).any() and not np.isnan(dv).any()
    # every head: total mass of dV (f32 sums of bf16-rounded rows; 4096 rows of magnitude ~1 summed: tolerance on the sum)
    mass_got, mass_ref = dv.astype(np.float64).sum(2), go.astype(np.float64).sum(2)
    err = float(np.abs(mass_got - mass_ref).max())
    say("   sum_j dV_j = sum_i dO_i over all %d heads: max-abs err %.3e (sums of magnitude %.1f)" % (B * H, err, float(np.abs(mass_ref).max())))
    assert err <= 2e-2 * float(np.abs(mass_ref).max())
    # three slices against the oracle; in them also: the last key meets the last query only -> dV_last = P_last,last * dO_last
    x_last = (q[:, :, -1].astype(np.float64) * k[:, :, -1]).sum(-1) / np.sqrt(D)
    for (b, h) in [(0, 0), (B - 1, H - 1), (3, 7)]:
        rq, rk, rv = BW.sdpa_backward(q[b, h], k[b, h], v[b, h], go[b, h], causal=True)
        for name, got, ref in (("dq", dq[b, h], rq), ("dk", dk[b, h], rk), ("dv", dv[b, h], rv)):
            e = float(np.abs(got - ref).max() / np.abs(ref).max())
            say("   slice (%d, %d) %s: max-abs err / max|ref| %.3e" % (b, h, name, e))
            assert e <= 2e-2
        lse_row = BW.logsumexp(q[b, h], k[b, h], causal=True)[-1]
        p_last = np.exp(x_last[b, h] - lse_row)
        assert np.abs(dv[b, h, -1] - p_last * go[b, h, -1]).max() <= 2e-2 * max(1.0, float(np.abs(p_last * go[b, h, -1]).max()))


@pytest.mark.parametrize("dt", [capi.BF16, capi.F32], ids=["bf16", "f32"])
def test_one_long_sequence_forward_and_backward(gpu, dt):
    """131072 tokens, two query heads on one KV head, bf16 and f32, causal: byte offsets inside a head reach 2^25 (f32: 2^26), a head's scores
    2^34 pairs, a workgroup walks up to 2048 tiles.  In float64 on the host, from what a row or a key needs alone: output and dQ
    of sampled rows; dK and dV of sampled keys among the last 2048 (their rows' normalisers cost a 2048 x 131072 product).  For
    all of it, identities that need no oracle: the column sums of dV are those of dO (every probability row sums to one), and
    sum_j <dK_j, k_j> = sum_i <dQ_i, q_i> (both are scale * sum_ij dS_ij <q_i, k_j>)."""
    B, Hq, Hkv, S, D = 1, 2, 1, 131072, 128
    eps = 2.0 ** -9 if dt == capi.BF16 else 2.0 ** -18          # (f32: roundings of sums of up to 131072 terms)
    say("one long sequence: %s causal S=131072, 2 query heads on 1 KV head, D=128" % dtypes.NAMES[dt])
    q, go = gen(70, (B, Hq, S, D), dt), gen(73, (B, Hq, S, D), dt)
    k, v = gen(71, (B, Hkv, S, D), dt), gen(72, (B, Hkv, S, D), dt)
    out, dq, dk, dv = host.sdpa_backward(q, k, v, go, dt, causal=True)
    scale = 1.0 / np.sqrt(D)
    k64, v64 = k[0, 0].astype(np.float64), v[0, 0].astype(np.float64)
    q64, go64 = q[0].astype(np.float64), go[0].astype(np.float64)
    worst = {"o": 0.0, "dq": 0.0, "dk": 0.0, "dv": 0.0}          # (gradients: largest error over the sampled rows or keys ...
    largest = {"dq": 0.0, "dk": 0.0, "dv": 0.0}                # ... against the largest reference magnitude among them)
    for h in range(Hq):
        for i in [0, 1, 63, 64, 255, 256, 4097, 65535, 65536, 100003, S - 2, S - 1]:
            s = (k64[:i + 1] @ q64[h, i]) * scale
            p = np.exp(s - s.max())
            p /= p.sum()
            o_ref = p @ v64[:i + 1]
            worst["o"] = max(worst["o"], float(np.abs(out[0, h, i] - o_ref).max()))
            ds = p * (v64[:i + 1] @ go64[h, i] - float(o_ref @ go64[h, i]))
            dq_ref = (ds @ k64[:i + 1]) * scale
            worst["dq"], largest["dq"] = max(worst["dq"], float(np.abs(dq[0, h, i] - dq_ref).max())), max(largest["dq"], float(np.abs(dq_ref).max()))
    T = 2048                                   # the last T rows: normalisers and D_i = <dO_i, O_i> in float64
    lse, delta = np.empty((Hq, T)), np.empty((Hq, T))
    for h in range(Hq):
        s = (q64[h, S - T:] @ k64.T) * scale
        s[np.arange(S - T, S)[:, None] < np.arange(S)[None, :]] = -np.inf
        m = s.max(axis=1)
        e = np.exp(s - m[:, None])
        lse[h] = m + np.log(e.sum(axis=1))
        delta[h] = np.einsum("id,id->i", (e / e.sum(axis=1)[:, None]) @ v64, go64[h, S - T:])
    for j in [S - T, S - 1500, S - 129, S - 128, S - 33, S - 1]:
        dk_ref, dv_ref = np.zeros(D), np.zeros(D)
        for h in range(Hq):
            r = j - (S - T)
            p = np.exp((q64[h, j:] @ k64[j]) * scale - lse[h, r:])
            dv_ref += p @ go64[h, j:]
            dk_ref += ((p * (go64[h, j:] @ v64[j] - delta[h, r:])) @ q64[h, j:]) * scale
        worst["dk"], largest["dk"] = max(worst["dk"], float(np.abs(dk[0, 0, j] - dk_ref).max())), max(largest["dk"], float(np.abs(dk_ref).max()))
        worst["dv"], largest["dv"] = max(worst["dv"], float(np.abs(dv[0, 0, j] - dv_ref).max())), max(largest["dv"], float(np.abs(dv_ref).max()))
    for name in largest:
        worst[name] /= largest[name]
    say("one long sequence: worst output error %.3e; gradients relative to the largest among the sampled rows or keys: dq %.3e dk %.3e dv %.3e"
        % (worst["o"], worst["dq"], worst["dk"], worst["dv"]))
    assert worst["o"] <= TOL[dt]
    assert max(worst["dq"], worst["dk"], worst["dv"]) <= TOL[dt]
    # the identities, with room for the roundings of 131072 bf16 rows adding up like a random walk
    dv64, dk64, dq64 = dv[0, 0].astype(np.float64), dk[0, 0].astype(np.float64), dq[0].astype(np.float64)
    sums, want = dv64.sum(axis=0), go64.sum(axis=(0, 1))
    say("one long sequence: column sums of dV against those of dO: worst %.3e" % np.abs(sums - want).max())
    # (bf16: a row's probabilities are rounded before the product with dO: they sum to one within 2^-9, and the rows' errors,
    #  each times a dO of order one, add up like a random walk)
    assert np.abs(sums - want).max() <= eps * np.sqrt(Hq * S) * np.abs(go64).max()
    tk, tq = np.einsum("jd,jd->j", dk64, k64), np.einsum("hid,hid->hi", dq64, q64)
    say("one long sequence: sum <dK, k> = %.6e, sum <dQ, q> = %.6e" % (tk.sum(), tq.sum()))
    assert abs(tk.sum() - tq.sum()) <= 8 * eps * (np.sqrt((tk ** 2).sum()) + np.sqrt((tq ** 2).sum()))


@pytest.mark.parametrize("dt", [capi.BF16, capi.F32], ids=["bf16", "f32"])
@pytest.mark.parametrize("shape", [(4096, 8, 49, 32, False), (60000, 1, 40, 64, True)], ids=["windows_49x32", "batch_60000"])
def test_very_many_small_heads(gpu, dt, shape):
    """Tens of thousands of small heads (window attention: 4096 windows x 8 heads of 49 tokens, head dimension 32; a batch of
    60000, just under the limit of a launch): work lists of 32768 - 60000 items on every kernel, forward and backward, with
    sampled heads - first, last, middle, random - against the oracles."""
    from oracle import sdpa_backward as BW
    B, H, S, D, causal = shape
    say("very many small heads: %s B=%d H=%d S=%d D=%d causal=%s" % (dtypes.NAMES[dt], B, H, S, D, causal))
    r = np.random.Generator(np.random.PCG64(75))
    q, k, v, go = (dtypes.round_to(r.standard_normal((B, H, S, D), dtype=np.float32), dt) for _ in range(4))
    out, dq, dk, dv = host.sdpa_backward(q, k, v, go, dt, causal=causal)
    for b, h in ((0, 0), (B - 1, H - 1), (B // 2, H // 2), (int(r.integers(0, B)), int(r.integers(0, H))), (B - 9, 0), (7, H - 1)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        ref = O.sdpa(q[sl], k[sl], v[sl], causal=causal)
        assert float(np.abs(out[sl] - ref).max()) <= TOL[dt], "output of head (%d, %d)" % (b, h)
        for name, g, r_ in zip(("dq", "dk", "dv"), (dq, dk, dv), BW.sdpa_backward(q[sl], k[sl], v[sl], go[sl], causal=causal)):
            err = float(np.abs(g[sl] - r_).max() / np.abs(r_).max())
            assert err <= TOL[dt], "%s of head (%d, %d): %.3e" % (name, b, h, err)
