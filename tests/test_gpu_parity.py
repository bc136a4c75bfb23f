"""Parity of the HIP kernels (through the C ABI) with the CPU oracle.

Tolerances (max-abs error against the f32 oracle run on the same inputs, which
for f16/bf16 are first rounded to the storage dtype):
    f32  1e-5        f16 / bf16  2e-2
"""
import sys

import numpy as np
import pytest

from incin_amd import capi, dtypes, host
from oracle import oracle as O

pytestmark = pytest.mark.gpu

TOL = {capi.F32: 1e-5, capi.F16: 2e-2, capi.BF16: 2e-2}
SEED0 = 20261125


def say(msg):
    print(msg, file=sys.stderr, flush=True)


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def inputs(seed, B, Hq, Hkv, Sq, Skv, D, Dv, dtype):
    r = rng(seed)
    q = dtypes.round_to(r.standard_normal((B, Hq, Sq, D), dtype=np.float32), dtype)
    k = dtypes.round_to(r.standard_normal((B, Hkv, Skv, D), dtype=np.float32), dtype)
    v = dtypes.round_to(r.standard_normal((B, Hkv, Skv, Dv), dtype=np.float32), dtype)
    return q, k, v


def oracle_full(q, k, v, G=1, **kw):
    """Oracle on [B,Hq,..] operands; GQA is expressed the way the reference expresses it:
    q [B,Hkv,G,S,D] against k, v [B,Hkv,1,S,D]."""
    B, Hq, Sq, D = q.shape
    Hkv = k.shape[1]
    q5 = q.reshape(B, Hkv, G, Sq, D)
    k5, v5 = k[:, :, None], v[:, :, None]
    if "kv_lens" in kw and kw["kv_lens"] is not None:
        kw = dict(kw, kv_lens=np.asarray(kw["kv_lens"], np.int32).reshape(B, 1, 1))
    if kw.get("mask") is not None:
        m = np.asarray(kw["mask"], np.float32)
        if m.ndim == 4:                                    # [B|1, Hq|1, Sq, Skv] -> [B|1, Hkv|1, G|1, Sq, Skv]
            if m.shape[1] == 1:
                m = m[:, :, None]
            else:
                m = m.reshape(m.shape[0], Hkv, G, m.shape[2], m.shape[3])
        kw = dict(kw, mask=m)
    out = O.sdpa(q5, k5, v5, **kw)
    return out.reshape(B, Hq, Sq, -1)


def check(got, ref, tol, what):
    assert got.shape == ref.shape, what
    nan_g, nan_r = np.isnan(got), np.isnan(ref)
    assert np.array_equal(nan_g, nan_r), "%s: NaN pattern differs (%d vs %d)" % (what, nan_g.sum(), nan_r.sum())
    err = np.abs(np.where(nan_r, 0, got) - np.where(nan_r, 0, ref)).max() if got.size else 0.0
    say("%s: max-abs err %.3e (tol %.0e)" % (what, err, tol))
    assert err <= tol, "%s: max-abs error %.3e > %.0e" % (what, err, tol)


def test_device_is_gfx950(gpu):
    info = gpu.device_info(0)
    say("device: %s %s CUs=%d clk=%d kHz" % (info.name.decode(), info.arch.decode(), info.compute_units, info.clock_khz))
    assert info.arch.decode().startswith("gfx950")
    assert info.wavefront_size == 64
    with pytest.raises(capi.RocmError) as e:
        gpu.device_info(99)
    assert e.value.code == capi.EDEVICE


def test_buffer_round_trip(gpu):
    x = rng(1).standard_normal(100003).astype(np.float32)
    buf = capi.DeviceBuffer.from_numpy(x)
    assert buf.ptr % 256 == 0
    assert np.array_equal(buf.to_numpy(np.float32, x.shape), x)
    buf.free()
    raw = dtypes.encode(x, capi.BF16)
    t = host.DeviceTensor.from_f32(x.reshape(1, 1, 1, -1), capi.BF16)
    assert np.array_equal(dtypes.encode(t.to_f32(), capi.BF16).reshape(-1), raw)


# ---- the two f32 benchmark configurations ------------------------------------------------

def test_config1_f32_single_head_noncausal(gpu):
    q, k, v = inputs(SEED0 + 0, 1, 1, 1, 128, 128, 64, 64, capi.F32)
    got, info = host.sdpa(q, k, v, capi.F32, scale=0.125, return_info=True)
    assert info["impl"] == capi.IMPL_SPLITKV_MFMA       # one 128-row block: the f32 split-KV kernel, 32 rows per workgroup
    ref = O.sdpa(q, k, v, scale=0.125)
    check(got, ref, 1e-5, "C1 f32 B1 H1 S128 D64")
    check(host.sdpa(q, k, v, capi.F32, scale=0.125, impl=capi.IMPL_MFMA), ref, 1e-5, "C1, the IEEE-f32 matrix-core prefill kernel")
    check(host.sdpa(q, k, v, capi.F32, scale=0.125, impl=capi.IMPL_GENERIC), ref, 1e-5, "C1, generic kernel")
    assert np.abs(ref - O.brute_f64(q, k, v, scale=0.125)).max() < 1e-6


def test_config2_f32_multi_head_causal(gpu):
    q, k, v = inputs(SEED0 + 1, 4, 8, 8, 1024, 1024, 64, 64, capi.F32)
    got, info = host.sdpa(q, k, v, capi.F32, causal=True, return_info=True)
    assert info["impl"] == capi.IMPL_SPLITKV_MFMA       # 256 row blocks of 128 on 256 compute units: the f32 split-KV kernel
    mask = O.causal_additive_mask(1024, 1024)                       # the explicit 0/-inf tensor the CPU op is given
    ref = O.sdpa(q, k, v, mask=mask)
    check(got, ref, 1e-5, "C2 f32 B4 H8 S1024 D64 causal")
    check(host.sdpa(q, k, v, capi.F32, causal=True, impl=capi.IMPL_MFMA), ref, 1e-5, "C2, the IEEE-f32 matrix-core prefill kernel")
    check(host.sdpa(q, k, v, capi.F32, causal=True, impl=capi.IMPL_GENERIC), ref, 1e-5, "C2, generic kernel")
    # the same mask handed over as a dense additive tensor, as a caller of the reference's operator passes it, goes
    # through the mask path of either kernel
    got2, info = host.sdpa(q, k, v, capi.F32, mask=mask, return_info=True)
    assert info["impl"] == capi.IMPL_MFMA
    check(got2, ref, 1e-5, "C2, dense additive mask")
    got3 = host.sdpa(q[:1, :2], k[:1, :2], v[:1, :2], capi.F32, mask=mask, impl=capi.IMPL_GENERIC)
    check(got3, ref[:1, :2], 1e-5, "C2 slice, dense additive mask, generic kernel")


# ---- generic kernel: shapes, masks, dtypes ----------------------------------------------

@pytest.mark.parametrize("dtype", [capi.F32, capi.F16, capi.BF16])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, D, Dv
    (1, 1, 1, 1, 1, 1, 1),
    (2, 3, 3, 77, 131, 40, 72),
    (1, 4, 2, 65, 64, 128, 128),
    (2, 2, 1, 5, 300, 200, 256),
    (1, 2, 2, 130, 7, 16, 8),
])
def test_generic_shapes(gpu, dtype, shape):
    B, Hq, Hkv, Sq, Skv, D, Dv = shape
    q, k, v = inputs(100 + sum(shape), B, Hq, Hkv, Sq, Skv, D, Dv, dtype)
    for causal in (False, True):
        got = host.sdpa(q, k, v, dtype, causal=causal, impl=capi.IMPL_GENERIC)
        ref = oracle_full(q, k, v, G=Hq // Hkv, causal=causal)
        check(got, ref, TOL[dtype], "generic %s %r causal=%d" % (dtypes.NAMES[dtype], shape, causal))


@pytest.mark.parametrize("dtype", [capi.F32, capi.BF16])
def test_generic_dense_masks_and_lengths(gpu, dtype):
    B, Hq, Hkv, Sq, Skv, D = 2, 4, 2, 70, 90, 32
    q, k, v = inputs(7, B, Hq, Hkv, Sq, Skv, D, D, dtype)
    r = rng(8)
    for mshape in [(Sq, Skv), (1, Skv), (B, 1, Sq, Skv), (B, Hq, Sq, Skv), (1, Hq, 1, Skv)]:
        m = dtypes.round_to(r.standard_normal(mshape, dtype=np.float32), dtype)
        m = np.where(r.random(mshape) < 0.25, -np.inf, m).astype(np.float32)
        m[..., 0] = 0.0                                             # keep every row alive
        got = host.sdpa(q, k, v, dtype, mask=m, scale=0.3)
        ref = oracle_full(q, k, v, G=2, mask=m, scale=0.3)
        check(got, ref, TOL[dtype], "generic %s mask %r" % (dtypes.NAMES[dtype], mshape))
    lens = np.array([0, 37], np.int32)                              # batch 0 has no visible key: NaN rows, as the reference
    got = host.sdpa(q, k, v, dtype, kv_lens=lens, causal=True, impl=capi.IMPL_GENERIC)
    ref = oracle_full(q, k, v, G=2, kv_lens=lens, causal=True)
    assert np.isnan(ref[0]).all() and np.isfinite(ref[1]).all()
    check(got, ref, TOL[dtype], "generic %s kv_lens+causal" % dtypes.NAMES[dtype])
    m = np.zeros((Sq, Skv), np.float32)
    m[3, :] = -np.inf                                               # one fully masked row
    got = host.sdpa(q, k, v, dtype, mask=m)
    check(got, oracle_full(q, k, v, G=2, mask=m), TOL[dtype], "generic fully masked row")


def test_reference_golden_vectors_on_gpu(gpu):
    import json, os
    gold = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))
    g = gold["attention_heads"]
    q = np.array([c["q"] for c in g["cases"]], np.float32).reshape(1, 2, 2, 1)
    k = np.array([c["k"] for c in g["cases"]], np.float32).reshape(1, 2, 2, 1)
    v = np.array([c["v"] for c in g["cases"]], np.float32).reshape(1, 2, 2, 1)
    got = host.sdpa(q, k, v, capi.F32, scale=g["scale"]).reshape(-1)
    exp = np.array([c["expected"] for c in g["cases"]]).reshape(-1)
    assert np.abs(got - exp).max() <= g["tol"]
    ones = np.ones((1, 1, 2, 4), np.float32)
    got = host.sdpa(ones, ones, ones, capi.F32)
    assert got.shape == (1, 1, 2, 4) and np.abs(got - 1.0).max() <= gold["sdpa_ones"]["tol"]
    for case in gold["softmax"]["cases"]:
        x = np.array(case["x"], np.float32)
        got = host.sdpa(np.ones((1, 1, 1, 1), np.float32), x.reshape(1, 1, -1, 1),
                        np.eye(len(x), dtype=np.float32).reshape(1, 1, len(x), len(x)), capi.F32, scale=1.0)
        assert np.abs(got.reshape(-1) - np.array(case["expected"])).max() <= case["tol"]


# ---- MFMA prefill kernel --------------------------------------------------------------------

MFMA_IMPLS = [capi.IMPL_MFMA]


@pytest.mark.parametrize("impl", MFMA_IMPLS)
@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, D
    (1, 1, 1, 128, 128, 128),
    (2, 4, 4, 512, 512, 128),
    (1, 2, 2, 200, 333, 128),
    (2, 8, 2, 256, 256, 128),
    (1, 4, 1, 100, 1000, 64),
    (1, 2, 2, 384, 129, 64),
    (1, 1, 1, 17, 64, 128),
    (1, 2, 1, 1000, 1000, 128),
    (1, 1, 1, 300, 40, 64),
])
def test_mfma_prefill(gpu, dtype, shape, impl):
    B, Hq, Hkv, Sq, Skv, D = shape
    q, k, v = inputs(200 + sum(shape), B, Hq, Hkv, Sq, Skv, D, D, dtype)
    for causal in (False, True):
        got, info = host.sdpa(q, k, v, dtype, causal=causal, impl=impl, return_info=True)
        assert info["impl"] == impl
        ref = oracle_full(q, k, v, G=Hq // Hkv, causal=causal)
        check(got, ref, TOL[dtype], "mfma %s %r causal=%d" % (dtypes.NAMES[dtype], shape, causal))
        gen = host.sdpa(q, k, v, dtype, causal=causal, impl=capi.IMPL_GENERIC)
        check(got, gen, TOL[dtype], "mfma vs generic kernel %r causal=%d" % (shape, causal))


@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, D
    (1, 1, 1, 128, 128, 64),
    (2, 4, 4, 512, 512, 128),
    (1, 2, 2, 200, 333, 128),
    (2, 8, 2, 256, 256, 64),
    (1, 4, 1, 100, 1000, 64),
    (1, 2, 2, 384, 129, 128),
    (1, 1, 1, 17, 64, 128),
    (1, 2, 1, 1000, 1000, 64),
    (1, 1, 1, 300, 40, 64),
    (2, 3, 3, 1, 70, 128),
])
def test_f32_matrix_core_prefill(gpu, shape):
    """The IEEE-f32 matrix-core kernel on f32 operands - the reference's own dtype - against the oracle at 1e-5:
    no mask, causal, ragged key counts with a causal mask, and dense additive masks of several broadcast shapes."""
    B, Hq, Hkv, Sq, Skv, D = shape
    G = Hq // Hkv
    q, k, v = inputs(400 + sum(shape), B, Hq, Hkv, Sq, Skv, D, D, capi.F32)
    for causal in (False, True):
        got, info = host.sdpa(q, k, v, capi.F32, causal=causal, impl=capi.IMPL_MFMA, return_info=True)
        assert info["impl"] == capi.IMPL_MFMA
        check(got, oracle_full(q, k, v, G=G, causal=causal), 1e-5, "f32 mfma %r causal=%d" % (shape, causal))
    r = rng(sum(shape))
    lens = r.integers(0, Skv + 1, B).astype(np.int32)
    got = host.sdpa(q, k, v, capi.F32, causal=True, kv_lens=lens, impl=capi.IMPL_MFMA)
    check(got, oracle_full(q, k, v, G=G, causal=True, kv_lens=lens), 1e-5, "f32 mfma %r causal + kv_lens %s" % (shape, lens.tolist()))
    for mshape in [(Sq, Skv), (1, Skv), (B, 1, Sq, Skv), (B, Hq, Sq, Skv), (1, Hq, 1, Skv)]:
        m = r.standard_normal(mshape, dtype=np.float32)
        m = np.where(r.random(mshape) < 0.25, -np.inf, m).astype(np.float32)
        m[..., 0] = 0.0                                             # keep every row alive
        got, info = host.sdpa(q, k, v, capi.F32, mask=m, scale=0.3 / np.sqrt(D / 32), return_info=True)
        assert info["impl"] == capi.IMPL_MFMA
        check(got, oracle_full(q, k, v, G=G, mask=m, scale=0.3 / np.sqrt(D / 32)), 1e-5, "f32 mfma %r mask %r" % (shape, mshape))
    m = np.zeros((Sq, Skv), np.float32)
    m[Sq // 2, :] = -np.inf                                         # one fully masked row: NaN, as the reference
    got = host.sdpa(q, k, v, capi.F32, mask=m, impl=capi.IMPL_MFMA)
    check(got, oracle_full(q, k, v, G=G, mask=m), 1e-5, "f32 mfma fully masked row")
    got, lse = host.sdpa(q, k, v, capi.F32, causal=True, impl=capi.IMPL_MFMA, return_lse=True)
    _, lse_g = host.sdpa(q, k, v, capi.F32, causal=True, impl=capi.IMPL_GENERIC, return_lse=True)
    fin = np.isfinite(lse_g)                                        # rows without a visible key: -inf in both
    assert np.array_equal(np.isfinite(lse), fin) and np.all(lse[~fin] == -np.inf)
    assert not fin.any() or np.abs(lse[fin] - lse_g[fin]).max() <= 1e-5


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, D
    (2, 4, 2, 70, 90, 128),            # the shapes of the generic-kernel mask test, at the matrix-core head dimensions
    (1, 2, 2, 300, 333, 128),          # key count not a multiple of 4: element-wise mask loads
    (2, 4, 4, 512, 512, 64),
    (1, 2, 1, 1000, 1000, 128),
    (1, 1, 1, 17, 64, 64),
])
def test_mfma_prefill_dense_masks(gpu, dtype, shape):
    """A dense additive mask keeps a 16-bit request on the matrix-core kernel: random masks of every broadcast shape
    (values, -inf entries), the causal mask as the tensor full(-inf).triu(1) a caller of the reference builds (equal to
    the causal flag bit for bit where whole blocks are hidden or zero), a banded mask (hidden blocks on both sides),
    masks combined with the causal flag and key counts, and a fully masked row."""
    B, Hq, Hkv, Sq, Skv, D = shape
    G = Hq // Hkv
    q, k, v = inputs(500 + sum(shape), B, Hq, Hkv, Sq, Skv, D, D, dtype)
    r = rng(sum(shape))
    for mshape in [(Sq, Skv), (1, Skv), (B, 1, Sq, Skv), (B, Hq, Sq, Skv), (1, Hq, 1, Skv)]:
        m = dtypes.round_to(r.standard_normal(mshape, dtype=np.float32), dtype)
        m = np.where(r.random(mshape) < 0.25, -np.inf, m).astype(np.float32)
        m[..., 0] = 0.0                                             # keep every row alive
        got, info = host.sdpa(q, k, v, dtype, mask=m, scale=0.3 / np.sqrt(D / 32), return_info=True)
        assert info["impl"] == capi.IMPL_MFMA and info["workspace_bytes"] > 0
        check(got, oracle_full(q, k, v, G=G, mask=m, scale=0.3 / np.sqrt(D / 32)), TOL[dtype], "mfma %s %r mask %r" % (dtypes.NAMES[dtype], shape, mshape))
    cm = O.causal_additive_mask(Sq, Skv)
    got, info = host.sdpa(q, k, v, dtype, mask=cm, return_info=True)
    assert info["impl"] == capi.IMPL_MFMA
    check(got, oracle_full(q, k, v, G=G, causal=True), TOL[dtype], "mfma causal mask as a tensor")
    flagged = host.sdpa(q, k, v, dtype, causal=True, impl=capi.IMPL_MFMA)
    check(got, flagged, 8e-3, "causal tensor vs causal flag")
    band = np.where(np.abs(np.arange(Sq)[:, None] + (Skv - Sq) - np.arange(Skv)[None, :]) <= 100, 0.0, -np.inf).astype(np.float32)
    got = host.sdpa(q, k, v, dtype, mask=band)
    check(got, oracle_full(q, k, v, G=G, mask=band), TOL[dtype], "mfma banded mask")
    lens = r.integers(1, Skv + 1, B).astype(np.int32)
    m = dtypes.round_to(r.standard_normal((Sq, Skv), dtype=np.float32), dtype)
    got = host.sdpa(q, k, v, dtype, mask=m, causal=True, kv_lens=lens)
    full = np.broadcast_to(m, (B, Hq, Sq, Skv)) + cm + np.where(np.arange(Skv)[None, :] < lens[:, None], 0.0, -np.inf).astype(np.float32)[:, None, None, :]
    check(got, oracle_full(q, k, v, G=G, mask=full), TOL[dtype], "mfma mask + causal flag + kv_lens")
    m = np.zeros((Sq, Skv), np.float32)
    m[Sq // 2, :] = -np.inf
    check(host.sdpa(q, k, v, dtype, mask=m), oracle_full(q, k, v, G=G, mask=m), TOL[dtype], "mfma fully masked row")
    hidden = np.full((Sq, Skv), -np.inf, np.float32)                # the mask hides everything: NaN everywhere, as the reference
    assert np.isnan(host.sdpa(q, k, v, dtype, mask=hidden)).all()


@pytest.mark.parametrize("impl", MFMA_IMPLS)
def test_mfma_prefill_ragged_lengths(gpu, impl):
    B, Hq, Hkv, S, D = 3, 8, 2, 640, 128
    q, k, v = inputs(31, B, Hq, Hkv, S, S, D, D, capi.BF16)
    lens = np.array([640, 129, 0], np.int32)
    got = host.sdpa(q, k, v, capi.BF16, causal=True, kv_lens=lens, impl=impl)
    ref = oracle_full(q, k, v, G=4, causal=True, kv_lens=lens)
    check(got, ref, 2e-2, "mfma bf16 GQA causal + kv_lens")
    # padded keys == truncated keys
    trunc = host.sdpa(q[1:2, :, :, :], k[1:2, :, :129], v[1:2, :, :129], capi.BF16, impl=impl)
    padded = host.sdpa(q[1:2], k[1:2], v[1:2], capi.BF16, kv_lens=lens[1:2], impl=impl)
    check(padded, trunc, 1e-6, "mfma padded == truncated")


@pytest.mark.parametrize("impl", [capi.IMPL_AUTO, capi.IMPL_GENERIC] + MFMA_IMPLS)
@pytest.mark.parametrize("causal", [True, False])
def test_padded_queries(gpu, impl, causal):
    """q_lens declares query rows padding: rows below the length are what they are without it (bit for bit);
    rows at and beyond it are unspecified and not looked at."""
    B, Hq, Hkv, S, D = 4, 4, 2, 600, 128
    q, k, v = inputs(41, B, Hq, Hkv, S, S, D, D, capi.BF16)
    lens = np.array([600, 257, 64, 0], np.int32)          # full, inside a block, a block boundary, nothing
    say("padded queries: impl %d causal %s lens %s" % (impl, causal, lens.tolist()))
    plain = host.sdpa(q, k, v, capi.BF16, causal=causal, kv_lens=lens, impl=impl)
    got = host.sdpa(q, k, v, capi.BF16, causal=causal, kv_lens=lens, q_lens=lens, impl=impl)
    ref = oracle_full(q, k, v, G=2, causal=causal, kv_lens=lens)
    for b in range(B):
        n = int(lens[b])
        assert np.array_equal(got[b, :, :n], plain[b, :, :n]), "batch %d" % b
        if n:
            check(got[b:b + 1, :, :n], ref[b:b + 1, :, :n], 2e-2, "padded queries, batch %d" % b)
    # lengths of Sq and beyond change nothing at all
    same = host.sdpa(q, k, v, capi.BF16, causal=causal, kv_lens=lens, q_lens=np.full(B, S, np.int32), impl=impl)
    assert np.array_equal(np.nan_to_num(same, nan=7.0), np.nan_to_num(plain, nan=7.0))


@pytest.mark.parametrize("impl", [capi.IMPL_AUTO, capi.IMPL_GENERIC] + MFMA_IMPLS)
def test_row_normalisers(gpu, impl):
    """lse = log sum_j exp(x_ij) of every row, the forward's by-product that the backward needs."""
    from oracle import sdpa_backward as BW
    B, Hq, Hkv, Sq, Skv, D = 2, 4, 2, 300, 420, 128
    q, k, v = inputs(51, B, Hq, Hkv, Sq, Skv, D, D, capi.BF16)
    lens = np.array([420, 77], np.int32)
    for causal in (False, True):
        got, lse, info = host.sdpa(q, k, v, capi.BF16, causal=causal, kv_lens=lens, impl=impl, return_lse=True, return_info=True)
        want = BW.logsumexp(q.reshape(B, Hkv, 2, Sq, D), k[:, :, None], causal=causal, kv_lens=lens.reshape(B, 1, 1)).reshape(B, Hq, Sq)
        fin = np.isfinite(want)
        assert np.array_equal(np.isfinite(lse), fin) and np.all(lse[~fin] == -np.inf)
        err = float(np.abs(lse[fin] - want[fin]).max())
        say("row normalisers impl %d causal %s: max-abs err %.3e" % (impl, causal, err))
        assert err <= 2e-2                # the scores come from bf16 products of a Q pre-multiplied by the scale in bf16
        plain = host.sdpa(q, k, v, capi.BF16, causal=causal, kv_lens=lens, impl=info["impl"])
        assert np.array_equal(np.nan_to_num(got, nan=7.0), np.nan_to_num(plain, nan=7.0))


@pytest.mark.parametrize("case", [
    # impl, dtype, B, Hq, Hkv, Sq, Skv, D, splits
    (capi.IMPL_SPLITKV, capi.BF16, 2, 4, 2, 1, 1500, 128, 0), (capi.IMPL_SPLITKV, capi.BF16, 2, 4, 2, 2, 1500, 128, 1),
    (capi.IMPL_SPLITKV, capi.F32, 1, 4, 4, 1, 900, 64, 3),
    (capi.IMPL_SPLITKV_MFMA, capi.BF16, 2, 16, 2, 1, 1500, 128, 0), (capi.IMPL_SPLITKV_MFMA, capi.F16, 2, 16, 2, 3, 1500, 128, 1),
    (capi.IMPL_SPLITKV_MFMA, capi.BF16, 1, 8, 1, 9, 700, 64, 4),
    (capi.IMPL_MFMA, capi.BF16, 1, 4, 2, 100, 4500, 128, 0), (capi.IMPL_MFMA, capi.F32, 1, 2, 2, 70, 4200, 64, 3),
])
def test_row_normalisers_from_split_launches(gpu, case):
    """The same by-product from the launches that split the key axis - the split-KV kernels (their combine pass, or the
    kernel itself with one split) and the prefill kernels over key splits - with a sequence that ends inside a split and
    one without keys."""
    from oracle import sdpa_backward as BW
    impl, dtype, B, Hq, Hkv, Sq, Skv, D, splits = case
    G = Hq // Hkv
    q, k, v = inputs(61 + Skv, B, Hq, Hkv, Sq, Skv, D, D, dtype)
    lens = np.array([Skv - 13, 0][:B], np.int32)
    got, lse, info = host.sdpa(q, k, v, dtype, causal=True, kv_lens=lens, impl=impl, num_splits=splits, return_lse=True, return_info=True)
    assert info["impl"] == impl
    say("row normalisers: impl %d dtype %d, %d splits" % (impl, dtype, info["splits"]))
    want = BW.logsumexp(q.reshape(B, Hkv, G, Sq, D), k[:, :, None], causal=True, kv_lens=lens.reshape(B, 1, 1)).reshape(B, Hq, Sq)
    fin = np.isfinite(want)
    assert np.array_equal(np.isfinite(lse), fin) and np.all(lse[~fin] == -np.inf)
    err = float(np.abs(lse[fin] - want[fin]).max())
    say("row normalisers from split launches: max-abs err %.3e" % err)
    assert err <= (2e-5 if dtype == capi.F32 else 2e-2)
    plain = host.sdpa(q, k, v, dtype, causal=True, kv_lens=lens, impl=impl, num_splits=splits)
    assert np.array_equal(np.nan_to_num(got, nan=7.0), np.nan_to_num(plain, nan=7.0))
    check(got, oracle_full(q, k, v, G=G, causal=True, kv_lens=lens), TOL[dtype], "output beside the row normalisers")


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16, capi.F32])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, D, causal, key counts
    (1, 8, 2, 300, 5000, 128, True, None),          # a chunk of a long prompt: 24 workgroups, the keys supply the rest
    (1, 4, 4, 128, 4608, 128, False, None),
    (2, 2, 1, 77, 9000, 128, True, [9000, 4100]),   # the second sequence ends inside a split
    (1, 6, 3, 200, 4500, 64, True, None),           # head dimension 64
    (1, 2, 2, 130, 4096, 128, True, [300]),         # most splits see no key at all
    (1, 4, 2, 200, 4500, 256, True, None),          # the prefill kernel for head dimensions above 128 (16-bit)
    (2, 2, 2, 130, 4200, 160, True, [4200, 1000]),
])
def test_prefill_with_the_keys_split(gpu, dtype, shape):
    """The matrix-core prefill kernels (16-bit and f32) over splits of the key axis + combine (what AUTO does for launches with few row blocks
    over many keys): against the oracle with the library's split count and forced ones, and against the unsplit launch."""
    B, Hq, Hkv, Sq, Skv, D, causal, lens = shape
    if D > 128 and dtype == capi.F32:
        pytest.skip("f32 has no prefill kernel above 128 (the split-KV kernel's 256 instance takes those launches)")
    q, k, v = inputs(1200 + Sq + Skv, B, Hq, Hkv, Sq, Skv, D, D, dtype)
    lens = None if lens is None else np.asarray(lens, np.int32)
    ref = oracle_full(q, k, v, G=Hq // Hkv, causal=causal, kv_lens=lens)
    whole, info = host.sdpa(q, k, v, dtype, causal=causal, kv_lens=lens, impl=capi.IMPL_MFMA, num_splits=1, return_info=True)
    assert info["splits"] == 1
    for splits in (0, 2, 5, 13):
        say("prefill with the keys split: %s %r splits=%d" % (dtypes.NAMES[dtype], shape, splits))
        got, info = host.sdpa(q, k, v, dtype, causal=causal, kv_lens=lens, impl=capi.IMPL_MFMA, num_splits=splits, return_info=True)
        assert info["impl"] == capi.IMPL_MFMA and info["splits"] > 1 and info["workspace_bytes"] > 0
        check(got, ref, TOL[dtype], "prefill, keys split %d ways" % info["splits"])
        check(got, whole, 8e-3 if dtype != capi.F32 else 2e-6, "split vs whole")
    if D > 128:        # (AUTO keeps launches this small on the split-KV kernel: the test below)
        return
    got, info = host.sdpa(q, k, v, dtype, causal=causal, kv_lens=lens, return_info=True)      # AUTO comes to the same launch
    assert info["impl"] == capi.IMPL_MFMA and info["splits"] > 1


def test_auto_splits_the_keys_of_a_wide_prefill_launch_that_fills_the_device(gpu):
    """Head dimensions above 128: a chunk of a long prompt goes to the prefill kernel with its keys split when the splits
    give every compute unit a workgroup (64 row blocks x 8 splits here), and stays on the split-KV kernel when they do not
    (8 row blocks).  Both against the split-KV kernel pinned (itself against the oracle in test_head_dimensions_above_128)."""
    for Hq, Hkv, Sq, Skv, want in ((32, 8, 256, 16384, capi.IMPL_MFMA), (8, 8, 128, 8192, capi.IMPL_SPLITKV_MFMA)):
        q, k, v = inputs(1300 + Hq, 1, Hq, Hkv, Sq, Skv, 256, 256, capi.BF16)
        got, info = host.sdpa(q, k, v, capi.BF16, causal=True, return_info=True)
        assert info["impl"] == want, info
        if want == capi.IMPL_MFMA:
            assert info["splits"] > 1 and info["workspace_bytes"] > 0
        other = host.sdpa(q, k, v, capi.BF16, causal=True, impl=capi.IMPL_SPLITKV_MFMA)
        check(got, other, 8e-3, "prefill kernel for 256 with split keys against the split-KV kernel")
        rows = np.array([[0, 0], [Hq - 1, Sq - 1], [Hq // 2, Sq // 2], [1, 31]])
        ref = O.sdpa_rows(q.reshape(1, Hkv, Hq // Hkv, Sq, 256), k[:, :, None], v[:, :, None], rows, causal=True)
        assert np.abs(got.reshape(Hq, Sq, 256)[rows[:, 0], rows[:, 1]] - ref).max() <= TOL[capi.BF16]


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16], ids=lambda x: dtypes.NAMES[x])
@pytest.mark.parametrize("rows", ["128", "256"])
@pytest.mark.parametrize("D", [128, 64])
def test_mask_values_through_lds(gpu, dtype, rows, D, monkeypatch):
    """A 16-bit mask whose rows can be copied 16 bytes at a time (unit key stride, a key count that is a multiple of 8, aligned
    rows) reaches the prefill kernel's scores through LDS, a tile ahead of its use; tiles with values, tiles of zeros and
    tiles with hidden blocks all go through the pipelined loop.  Against the oracle: values everywhere, a distance bias under
    the causal triangle, a band, blocks of all three kinds at random, rows broadcast over queries, masks in which some blocks
    of 128 rows are all limits (computed by the launch before, so that half of a 256-row workgroup has nothing to do) and
    others carry values, on top of the causal flag and key counts, S_q not a multiple of the blocks; both workgroup forms."""
    monkeypatch.setenv("INCIN_ROCM_PREFILL_BLOCK_ROWS", rows)
    tol = TOL[dtype]
    r = rng(SEED0 + 140 + D)
    B, Hq, Hkv, Sq, Skv = 2, 4, 2, 600, 704
    q, k, v = inputs(3200 + D, B, Hq, Hkv, Sq, Skv, D, D, dtype)
    NEG = -np.inf
    causal = O.causal_additive_mask(Sq, Skv).reshape(1, 1, Sq, Skv)
    dist = (np.arange(Sq)[:, None] + (Skv - Sq) - np.arange(Skv)[None, :]).astype(np.float32)
    cases = []
    cases.append(("values everywhere [B,Hq,Sq,Skv]", r.standard_normal((B, Hq, Sq, Skv), dtype=np.float32), {}))
    slopes = (0.5 ** np.arange(1, Hq + 1, dtype=np.float32))[:, None, None]
    cases.append(("distance bias under the causal triangle [1,Hq,Sq,Skv]", np.where(dist >= 0, -dist[None] * slopes, NEG)[None].astype(np.float32), {}))
    cases.append(("a band of 150 keys with a bias inside [Sq,Skv]", np.where((dist >= 0) & (dist < 150), -0.01 * dist, NEG).astype(np.float32), {}))
    kinds = r.integers(0, 3, size=(1, Hq, (Sq + 31) // 32, (Skv + 31) // 32))
    kinds[..., 0] = 1                                                                      # every row keeps visible keys
    big = np.repeat(np.repeat(kinds, 32, axis=2), 32, axis=3)[:, :, :Sq, :Skv]
    cases.append(("blocks hidden / zero / valued at random [1,Hq,Sq,Skv]", np.where(big == 0, NEG, np.where(big == 1, 0.0, r.standard_normal((1, Hq, Sq, Skv), dtype=np.float32))).astype(np.float32), {}))
    cases.append(("one row of values for every query [B,1,1,Skv]", r.standard_normal((B, 1, 1, Skv), dtype=np.float32), {}))
    mixed = np.broadcast_to(causal, (1, Hq, Sq, Skv)).copy()
    mixed[0, :, 128:256] += r.standard_normal((Hq, 128, Skv), dtype=np.float32)           # rows 128..255 carry values, the blocks around them are limits
    mixed[0, 1, 384:512, :40] = -2.0
    cases.append(("causal, with blocks of 128 rows that carry values [1,Hq,Sq,Skv]", mixed, {}))
    cases.append(("values under a causal flag and key counts", r.standard_normal((Sq, Skv), dtype=np.float32), dict(causal=True, kv_lens=np.array([704, 68], np.int32))))
    for what, m, kw in cases:
        say("mask values through LDS: %s, %s rows, D=%d, %s" % (dtypes.NAMES[dtype], rows, D, what))
        m = dtypes.round_to(np.ascontiguousarray(m), dtype)
        got, info = host.sdpa(q, k, v, dtype, mask=m, impl=capi.IMPL_MFMA, return_info=True, **kw)
        assert info["impl"] == capi.IMPL_MFMA
        full = np.broadcast_to(m, (B, Hq, Sq, Skv)).copy()             # (the oracle takes one mask: the flag and the counts folded in)
        if kw.get("causal"):
            full += causal
        if kw.get("kv_lens") is not None:
            full += np.where(np.arange(Skv)[None, :] < kw["kv_lens"][:, None], 0.0, NEG).astype(np.float32)[:, None, None, :]
        check(got, oracle_full(q, k, v, G=Hq // Hkv, mask=full), tol, what)


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16], ids=lambda x: dtypes.NAMES[x])
@pytest.mark.parametrize("rows", ["128", "256"])
@pytest.mark.parametrize("D", [128, 64, 256])
def test_mask_tensors_whose_rows_are_zeros_then_minus_infinity(gpu, dtype, rows, D, monkeypatch):
    """A mask tensor whose every row is n zeros followed by -inf - the causal mask as the reference's callers build it, a
    key-padding mask, their sum - says nothing its row limits do not.  The 16-bit prefill launch writes a limit per mask row
    and runs the blocks of rows that all have one as a launch without a mask tensor does, the others from the mask's flags
    and values; every block is computed by exactly one of the two.  Against the oracle given the tensor: masks that are all
    limits, masks where some blocks are and some are not (a bias in a few rows), limits of 0 (rows that see nothing: NaN)
    and of Skv, rows broadcast over queries / heads / batch, on top of a causal flag and key counts, S_q not a multiple of
    the blocks, both workgroup forms."""
    monkeypatch.setenv("INCIN_ROCM_PREFILL_BLOCK_ROWS", rows)
    tol = TOL[dtype]
    r = rng(SEED0 + 120 + D)
    B, Hq, Hkv, Sq, Skv = 2, 4, 2, 600, 700
    q, k, v = inputs(3100 + D, B, Hq, Hkv, Sq, Skv, D, D, dtype)
    NEG = -np.inf
    causal = O.causal_additive_mask(Sq, Skv).reshape(1, 1, Sq, Skv)                       # aligned to the last key
    cases = []
    cases.append(("the causal tensor", causal, {}))
    pad = np.zeros((B, 1, 1, Skv), np.float32)
    pad[0, ..., 650:] = NEG
    pad[1, ..., 90:] = NEG
    cases.append(("key padding [B,1,1,Skv]", pad, {}))
    cases.append(("causal + key padding [B,1,Sq,Skv]", causal + pad, {}))
    lims = r.integers(0, Skv + 1, size=(B, Hq, Sq))                                        # any limit per row, 0 and Skv among them
    lims[0, 0, :5] = 0
    lims[1, 3, 300:310] = Skv
    anyl = np.where(np.arange(Skv)[None, None, None, :] < lims[..., None], 0.0, NEG).astype(np.float32)
    cases.append(("a limit of its own per row [B,Hq,Sq,Skv]", anyl, {}))
    mixed = np.broadcast_to(causal, (1, Hq, Sq, Skv)).copy()
    mixed[0, 1, 130:140, :20] = -1.5                                                       # head 1: rows 130..139 carry a bias: their block reads the mask
    mixed[0, 2, 599, 100] = NEG                                                            # head 2: a hole in the last row
    mixed[0, 3, 300, 400:] = 0.0                                                           # head 3: one row sees everything (a limit, too)
    cases.append(("causal with a few rows that are not limits [1,Hq,Sq,Skv]", mixed, {}))
    cases.append(("key padding under a causal flag and key counts", pad, dict(causal=True, kv_lens=np.array([700, 60], np.int32))))
    for what, m, kw in cases:
        say("limit masks: %s, %s rows, D=%d, %s" % (dtypes.NAMES[dtype], rows, D, what))
        m = dtypes.round_to(np.ascontiguousarray(m), dtype)
        got, lse, info = host.sdpa(q, k, v, dtype, mask=m, impl=capi.IMPL_MFMA, return_info=True, return_lse=True, **kw)
        assert info["impl"] == capi.IMPL_MFMA
        full = np.broadcast_to(m, (B, Hq, Sq, Skv)).copy()             # (the oracle takes one mask: the flag and the counts folded in)
        if kw.get("causal"):
            full += causal
        if kw.get("kv_lens") is not None:
            full += np.where(np.arange(Skv)[None, :] < kw["kv_lens"][:, None], 0.0, NEG).astype(np.float32)[:, None, None, :]
        check(got, oracle_full(q, k, v, G=Hq // Hkv, mask=full), tol, what)
        _, lse_g = host.sdpa(q, k, v, dtype, mask=m, impl=capi.IMPL_GENERIC, return_lse=True, **kw)
        fin = np.isfinite(lse_g)
        assert np.array_equal(np.isfinite(lse), fin) and np.max(np.abs(lse[fin] - lse_g[fin])) < 2e-2, what
    # the causal tensor and the causal flag are the same computation row for row
    flag = host.sdpa(q, k, v, dtype, causal=True, impl=capi.IMPL_MFMA)
    tens = host.sdpa(q, k, v, dtype, mask=dtypes.round_to(causal, dtype), impl=capi.IMPL_MFMA)
    assert np.array_equal(flag, tens, equal_nan=True)


@pytest.mark.parametrize("shape", [(2, 3, 3, 300, 400, 64), (1, 4, 2, 256, 256, 128), (2, 2, 2, 130, 500, 128)],
                         ids=["one_head_per_kv_head", "groups_of_whole_blocks", "a_ragged_last_block"])
def test_f32_mask_tensors_whose_rows_are_zeros_then_minus_infinity(gpu, shape):
    """f32, small launches: the 128-row blocks whose mask rows all have a limit are computed by the f32 split-KV kernel from
    the limits (the kernel AUTO gives such launches when there is no mask tensor), the others by the prefill kernel's
    dense-mask launch that follows.  Against the oracle at 1e-5; the causal tensor must reproduce the causal flag through
    the split-KV kernel bit for bit - which also says the limit launch is the one that ran."""
    B, Hq, Hkv, Sq, Skv, D = shape
    dt = capi.F32
    q, k, v = inputs(3200 + Sq + D, B, Hq, Hkv, Sq, Skv, D, D, dt)
    NEG = -np.inf
    causal = O.causal_additive_mask(Sq, Skv).reshape(1, 1, Sq, Skv)
    pad = np.zeros((B, 1, 1, Skv), np.float32)
    pad[0, ..., Skv - 30:] = NEG
    pad[-1, ..., 90:] = NEG
    mixed = np.broadcast_to(causal, (1, Hq, Sq, Skv)).copy()
    mixed[0, 0, 5:9, :3] = 0.75                                    # head 0, first block: rows with values - that block reads the mask
    mixed[0, Hq - 1, Sq - 1, 0] = NEG                              # last head, last block: a hole
    hidden = causal + pad
    hidden = np.broadcast_to(hidden, (B, 1, Sq, Skv)).copy()
    hidden[0, 0, 17] = NEG                                         # a row that sees nothing: limit 0, NaN
    for what, m in (("the causal tensor", causal), ("key padding", pad), ("causal with rows that are not limits", mixed),
                    ("causal + key padding, one row hidden entirely", hidden)):
        say("f32 limit masks %r: %s" % (shape, what))
        m = np.ascontiguousarray(m)
        got, lse, info = host.sdpa(q, k, v, dt, mask=m, return_info=True, return_lse=True)
        assert info["impl"] == capi.IMPL_MFMA
        check(got, oracle_full(q, k, v, G=Hq // Hkv, mask=m), TOL[dt], what)
        _, lse_g = host.sdpa(q, k, v, dt, mask=m, impl=capi.IMPL_GENERIC, return_lse=True)
        fin = np.isfinite(lse_g)
        assert np.array_equal(np.isfinite(lse), fin) and np.max(np.abs(lse[fin] - lse_g[fin])) < 2e-5, what
    flag = host.sdpa(q, k, v, dt, causal=True, impl=capi.IMPL_SPLITKV_MFMA, num_splits=1)
    tens = host.sdpa(q, k, v, dt, mask=causal)
    assert np.array_equal(flag, tens, equal_nan=True)


# ---- split-KV decode -----------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16, capi.F32])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, D
    (2, 4, 4, 1, 4096, 128),
    (1, 8, 2, 1, 3000, 128),
    (2, 8, 1, 1, 2048, 64),
    (1, 2, 2, 3, 1500, 128),
    (1, 16, 1, 1, 700, 64),
])
def test_decode_splitkv(gpu, dtype, shape):
    B, Hq, Hkv, Sq, Skv, D = shape
    q, k, v = inputs(300 + sum(shape), B, Hq, Hkv, Sq, Skv, D, D, dtype)
    ref = oracle_full(q, k, v, G=Hq // Hkv, causal=True)
    outs = []
    for splits in (0, 1, 3, 8):
        got, info = host.sdpa(q, k, v, dtype, causal=True, num_splits=splits, impl=capi.IMPL_SPLITKV, return_info=True)
        assert info["impl"] == capi.IMPL_SPLITKV
        check(got, ref, TOL[dtype], "decode %s %r splits=%d->%d" % (dtypes.NAMES[dtype], shape, splits, info["splits"]))
        outs.append(got)
    for o in outs[1:]:                                              # split-KV + combine == unsplit
        check(o, outs[1], 1e-5 if dtype == capi.F32 else 8e-3, "decode split-count invariance")


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, causal
    (2, 8, 2, 1, 4096, False),        # grouped-query decode, 4 rows per KV head
    (1, 32, 4, 1, 3000, False),       # 8 rows, ragged last tile
    (3, 16, 1, 1, 700, True),         # multi-query, 16 rows
    (1, 8, 2, 5, 1500, True),         # 20 rows per KV head with a causal edge among the 5 positions
    (1, 40, 1, 1, 333, False),        # 40 rows: two chunks of 32, the second mostly empty
    (2, 12, 4, 9, 1000, True),        # 27 rows
    (1, 4, 4, 40, 2500, True),        # one head per KV head, 40 positions: two chunks, causal
    (1, 8, 8, 1, 200, False),         # a single row per KV head, fewer keys than a split asks for
    (2, 64, 1, 1, 900, False),        # 64 rows: one workgroup of two 32-row blocks
    (1, 16, 2, 9, 1200, True),        # 72 rows per KV head: two chunks of 64, the second with 8 rows
    (1, 6, 2, 64, 1500, True),        # 192 rows per KV head: three chunks, causal over 64 positions
    (1, 4, 2, 8, 5, True),            # more positions than keys: the first three see none (NaN rows, as the reference)
])
@pytest.mark.parametrize("slots", ["2", "5"], ids=["two_slot_rings", "five_slot_rings"])
def test_decode_splitkv_matrix_cores(gpu, dtype, shape, slots, monkeypatch):
    """The matrix-core split-KV kernel against the oracle, with the split count left to the library, forced to one
    (the kernel writes the output itself) and forced to counts that leave ragged and empty last splits; and against
    the vector-ALU split-KV kernel where that one takes the shape.  Both forms of the 32-row instance on every shape:
    rings of two slots (two workgroups per compute unit; the library's choice for short splits) and of five."""
    monkeypatch.setenv("INCIN_ROCM_DECODE_SLOTS", slots)
    B, Hq, Hkv, Sq, Skv, causal = shape
    D = 128
    q, k, v = inputs(700 + sum(shape[:5]), B, Hq, Hkv, Sq, Skv, D, D, dtype)
    ref = oracle_full(q, k, v, G=Hq // Hkv, causal=causal)
    outs = []
    for splits in (0, 1, 3, 7, 40):
        say("matrix-core split-KV: %s %r splits=%d" % (dtypes.NAMES[dtype], shape, splits))
        got, info = host.sdpa(q, k, v, dtype, causal=causal, num_splits=splits, impl=capi.IMPL_SPLITKV_MFMA, return_info=True)
        assert info["impl"] == capi.IMPL_SPLITKV_MFMA
        check(got, ref, TOL[dtype], "matrix-core split-KV %s %r splits=%d->%d" % (dtypes.NAMES[dtype], shape, splits, info["splits"]))
        outs.append(got)
    for o in outs:
        check(o, outs[1], 8e-3, "matrix-core split-KV: split-count invariance")
    if (Hq // Hkv) * Sq <= 8:
        valu = host.sdpa(q, k, v, dtype, causal=causal, impl=capi.IMPL_SPLITKV)
        check(outs[0], valu, 8e-3, "matrix-core vs vector-ALU split-KV")


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16])
@pytest.mark.parametrize("slots", ["2", "5"], ids=["two_slot_rings", "five_slot_rings"])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, causal      (head dimension 64: blocks of 64 keys)
    (2, 8, 2, 1, 4096, False),
    (1, 14, 2, 1, 3001, False),       # 7 query heads per KV head, ragged last block
    (2, 16, 1, 3, 777, True),         # 48 rows: the 64-row instance, causal among the positions
    (1, 4, 4, 1, 130, False),         # two blocks and a bit
    (1, 2, 1, 40, 2000, True),        # 80 rows: two chunks of 64
])
def test_decode_splitkv_matrix_cores_d64(gpu, dtype, shape, slots, monkeypatch):
    """The same kernel at head dimension 64 (a slot holds 64 keys there) against the oracle and the vector-ALU kernel."""
    monkeypatch.setenv("INCIN_ROCM_DECODE_SLOTS", slots)
    B, Hq, Hkv, Sq, Skv, causal = shape
    D = 64
    q, k, v = inputs(900 + sum(shape[:5]), B, Hq, Hkv, Sq, Skv, D, D, dtype)
    ref = oracle_full(q, k, v, G=Hq // Hkv, causal=causal)
    lens = np.asarray([Skv - 1 - 37 * b for b in range(B)], np.int32)
    ref_l = oracle_full(q, k, v, G=Hq // Hkv, causal=causal, kv_lens=lens)
    for splits in (0, 1, 3, 9):
        say("matrix-core split-KV, D = 64: %s %r splits=%d" % (dtypes.NAMES[dtype], shape, splits))
        got, info = host.sdpa(q, k, v, dtype, causal=causal, num_splits=splits, impl=capi.IMPL_SPLITKV_MFMA, return_info=True)
        assert info["impl"] == capi.IMPL_SPLITKV_MFMA
        check(got, ref, TOL[dtype], "matrix-core split-KV D=64 %s %r splits=%d->%d" % (dtypes.NAMES[dtype], shape, splits, info["splits"]))
        got = host.sdpa(q, k, v, dtype, causal=causal, kv_lens=lens, num_splits=splits, impl=capi.IMPL_SPLITKV_MFMA)
        check(got, ref_l, TOL[dtype], "matrix-core split-KV D=64 with key counts")
    if (Hq // Hkv) * Sq <= 8:
        check(got, host.sdpa(q, k, v, dtype, causal=causal, kv_lens=lens, impl=capi.IMPL_SPLITKV), 8e-3, "matrix-core vs vector-ALU split-KV, D = 64")


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("slots", ["2", "5"], ids=["two_slot_rings", "five_slot_rings"])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, causal      (f32: chunks of 16 or 32 rows, blocks of 16 keys at D = 128 and 32 at D = 64)
    (2, 8, 2, 1, 4096, False),        # grouped-query decode, 4 rows per KV head
    (1, 32, 4, 1, 3000, False),       # 8 rows, ragged last block
    (3, 16, 1, 1, 700, True),         # multi-query, 16 rows: a full block of rows
    (1, 8, 2, 5, 1500, True),         # 20 rows: the 32-row instance, a causal edge among the 5 positions
    (1, 40, 1, 1, 333, False),        # 40 rows: two chunks of 32, the second with 8 rows
    (2, 12, 4, 9, 1000, True),        # 27 rows
    (1, 8, 8, 1, 200, False),         # a single row per KV head, fewer keys than a split asks for
    (1, 6, 2, 22, 1500, True),        # 66 rows per KV head: three chunks, causal over 22 positions
    (1, 4, 2, 8, 5, True),            # more positions than keys: the first three see none (NaN rows, as the reference)
])
def test_decode_splitkv_matrix_cores_f32(gpu, D, shape, slots, monkeypatch):
    """The f32 matrix-core split-KV kernel (IEEE-f32 matrix instructions) against the oracle at the f32 bar, with the
    split count left to the library, forced to one and forced to counts that leave ragged and empty last splits, with key
    counts per batch entry, and against the vector-ALU split-KV kernel where that one takes the shape; row normalisers
    from the one-split and the combined launches."""
    monkeypatch.setenv("INCIN_ROCM_DECODE_SLOTS", slots)
    B, Hq, Hkv, Sq, Skv, causal = shape
    dt = capi.F32
    q, k, v = inputs(1300 + D + sum(shape[:5]), B, Hq, Hkv, Sq, Skv, D, D, dt)
    ref = oracle_full(q, k, v, G=Hq // Hkv, causal=causal)
    lens = np.asarray([max(Skv - 1 - 37 * b, 0) for b in range(B)], np.int32)
    ref_l = oracle_full(q, k, v, G=Hq // Hkv, causal=causal, kv_lens=lens)
    outs = []
    for splits in (0, 1, 3, 7, 40):
        say("f32 matrix-core split-KV: D=%d %r splits=%d" % (D, shape, splits))
        got, info = host.sdpa(q, k, v, dt, causal=causal, num_splits=splits, impl=capi.IMPL_SPLITKV_MFMA, return_info=True)
        assert info["impl"] == capi.IMPL_SPLITKV_MFMA
        check(got, ref, TOL[dt], "f32 matrix-core split-KV D=%d %r splits=%d->%d" % (D, shape, splits, info["splits"]))
        outs.append(got)
        got = host.sdpa(q, k, v, dt, causal=causal, kv_lens=lens, num_splits=splits, impl=capi.IMPL_SPLITKV_MFMA)
        check(got, ref_l, TOL[dt], "f32 matrix-core split-KV with key counts, splits=%d" % splits)
    for o in outs:
        check(o, outs[1], 2e-6, "f32 matrix-core split-KV: split-count invariance")
    if (Hq // Hkv) * Sq <= 8:
        check(outs[0], host.sdpa(q, k, v, dt, causal=causal, impl=capi.IMPL_SPLITKV), 2e-6, "f32 matrix-core vs vector-ALU split-KV")


def test_decode_splitkv_matrix_cores_f32_scale_lse_auto(gpu):
    """A negative scale, the row normalisers (one split and combined) against the generic kernel's, and AUTO's choice for
    f32 grouped-query decode."""
    B, Hq, Hkv, Skv, D = 2, 16, 4, 1100, 128
    dt = capi.F32
    q, k, v = inputs(1733, B, Hq, Hkv, 1, Skv, D, D, dt)
    got = host.sdpa(q, k, v, dt, scale=-0.07, impl=capi.IMPL_SPLITKV_MFMA)
    check(got, oracle_full(q, k, v, G=4, scale=-0.07), TOL[dt], "f32 matrix-core split-KV negative scale")
    lens = np.array([1100, 0], np.int32)
    _, lse_ref = host.sdpa(q, k, v, dt, kv_lens=lens, impl=capi.IMPL_GENERIC, return_lse=True)
    for splits in (1, 4):
        got, lse = host.sdpa(q, k, v, dt, kv_lens=lens, impl=capi.IMPL_SPLITKV_MFMA, num_splits=splits, return_lse=True)
        check(got, oracle_full(q, k, v, G=4, kv_lens=lens), TOL[dt], "f32 matrix-core split-KV, an empty batch entry")
        assert np.all(np.isneginf(lse[1])) and np.all(np.isneginf(lse_ref[1]))
        assert np.max(np.abs(lse[0] - lse_ref[0])) < 2e-6
    got, info = host.sdpa(q, k, v, dt, return_info=True)
    assert info["impl"] == capi.IMPL_SPLITKV_MFMA           # 4 rows per KV head over 1100 keys, f32: AUTO's choice
    check(got, oracle_full(q, k, v, G=4), TOL[dt], "AUTO f32 grouped-query decode")
    got, info = host.sdpa(q[:, :4], k, v, dt, return_info=True)
    assert info["impl"] == capi.IMPL_SPLITKV_MFMA           # one row per KV head too (from 512 keys on)
    check(got, oracle_full(q[:, :4], k, v, G=1), TOL[dt], "AUTO f32 decode, one row per KV head")
    got, info = host.sdpa(q[:, :4], k[:, :, :300], v[:, :, :300], dt, return_info=True)
    assert info["impl"] == capi.IMPL_SPLITKV                # the shortest caches stay on the vector-ALU kernel
    check(got, oracle_full(q[:, :4], k[:, :, :300], v[:, :, :300], G=1), TOL[dt], "AUTO f32 decode over a short cache")


HEAD_DIMS_16 = [(96, 96), (80, 80), (40, 40), (8, 8), (112, 72), (128, 64), (64, 128), (32, 16), (120, 128)]
HEAD_DIMS_F32 = [(96, 96), (20, 20), (4, 4), (100, 36), (128, 64), (60, 128)]


@pytest.mark.parametrize("dtype,dims", [(dt, dd) for dt in (capi.BF16, capi.F16) for dd in HEAD_DIMS_16] +
                         [(capi.F32, dd) for dd in HEAD_DIMS_F32],
                         ids=lambda x: dtypes.NAMES[x] if isinstance(x, int) else "D%d_Dv%d" % x)
def test_head_dimensions_padded_into_the_matrix_core_kernels(gpu, dtype, dims):
    """Head dimensions up to 128 in whole 16-byte vectors, D and Dv not necessarily equal, run in the matrix-core kernels'
    64 or 128 instance (zeros on the way into LDS, stores cut at Dv): prefill with a causal mask, with key counts and with
    a dense mask, a chunk with the keys split, decode (one and several rows per KV head) through the split-KV kernels,
    row normalisers - each against the oracle, and AUTO must pick those kernels."""
    D, Dv = dims
    tol = TOL[dtype]
    # prefill, grouped queries, causal with S_q < S_kv, key counts
    B, Hq, Hkv, Sq, Skv = 2, 4, 2, 200, 333
    q, k, v = inputs(2100 + D + 3 * Dv, B, Hq, Hkv, Sq, Skv, D, Dv, dtype)
    lens = np.array([333, 97], np.int32)
    say("padded head dimensions: %s D=%d Dv=%d prefill" % (dtypes.NAMES[dtype], D, Dv))
    got, lse, info = host.sdpa(q, k, v, dtype, causal=True, kv_lens=lens, impl=capi.IMPL_MFMA, return_info=True, return_lse=True)
    check(got, oracle_full(q, k, v, G=2, causal=True, kv_lens=lens), tol, "prefill D=%d Dv=%d" % (D, Dv))
    got_a, info = host.sdpa(q, k, v, dtype, causal=True, kv_lens=lens, return_info=True)
    # (f32 launches this small go 32 rows per workgroup through the split-KV kernel)
    assert info["impl"] == (capi.IMPL_SPLITKV_MFMA if dtype == capi.F32 else capi.IMPL_MFMA)
    check(got_a, oracle_full(q, k, v, G=2, causal=True, kv_lens=lens), tol, "AUTO, prefill D=%d Dv=%d" % (D, Dv))
    _, lse_g = host.sdpa(q, k, v, dtype, causal=True, kv_lens=lens, impl=capi.IMPL_GENERIC, return_lse=True)
    assert np.max(np.abs(lse - lse_g)) < (2e-5 if dtype == capi.F32 else 2e-2)
    # a dense additive mask (values and hidden blocks)
    r = rng(5)
    m = (r.standard_normal((1, 1, Sq, Skv)) * 0.5).astype(np.float32)
    m[..., 64:160, 32:128] = -np.inf
    m = dtypes.round_to(m, dtype)
    got, info = host.sdpa(q, k, v, dtype, mask=m, return_info=True)
    assert info["impl"] == capi.IMPL_MFMA
    check(got, oracle_full(q, k, v, G=2, mask=m), tol, "dense mask D=%d Dv=%d" % (D, Dv))
    # a chunk of a long prompt: the library splits the keys, the combine pass cuts the partial rows at Dv
    q2, k2, v2 = inputs(2200 + D, 1, 4, 4, 128, 8192, D, Dv, dtype)
    got, info = host.sdpa(q2, k2, v2, dtype, causal=True, return_info=True)
    assert info["impl"] == capi.IMPL_MFMA and info["splits"] > 1
    check(got, oracle_full(q2, k2, v2, causal=True), tol, "prefill with the keys split, D=%d Dv=%d" % (D, Dv))
    # decode: one row per KV head and a short causal run of a group's heads, split counts chosen and forced
    for Hq3, Sq3 in ((2, 1), (8, 3)):
        q3, k3, v3 = inputs(2300 + D + Hq3, 2, Hq3, 2, Sq3, 1500, D, Dv, dtype)
        ref = oracle_full(q3, k3, v3, G=Hq3 // 2, causal=True)
        for splits in (0, 1, 5):
            say("padded head dimensions: decode Hq=%d Sq=%d splits=%d" % (Hq3, Sq3, splits))
            got, lse, info = host.sdpa(q3, k3, v3, dtype, causal=True, num_splits=splits, return_info=True, return_lse=True)
            assert info["impl"] == capi.IMPL_SPLITKV_MFMA
            check(got, ref, tol, "decode D=%d Dv=%d rows=%d splits=%d" % (D, Dv, Hq3 // 2 * Sq3, splits))
        _, lse_g = host.sdpa(q3, k3, v3, dtype, causal=True, impl=capi.IMPL_GENERIC, return_lse=True)
        assert np.max(np.abs(lse - lse_g)) < (2e-5 if dtype == capi.F32 else 2e-2)


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16, capi.F32], ids=lambda x: dtypes.NAMES[x])
@pytest.mark.parametrize("dims", [(256, 256), (192, 128), (160, 160), (136, 256), (64, 200)], ids=lambda x: "D%d_Dv%d" % x)
def test_head_dimensions_above_128(gpu, dtype, dims):
    """Head dimensions above 128: decode shapes (one and several rows per KV head) and every f32 shape go through the 256
    instance of the matrix-core split-KV kernels, 16-bit prefill shapes through the prefill kernel for 256 (and through the
    split-KV kernel when it is pinned) - causal, grouped queries, key counts, split counts chosen and forced, row
    normalisers - against the oracle."""
    D, Dv = dims
    tol = TOL[dtype]
    for (B, Hq, Hkv, Sq, Skv), split_list in (((2, 2, 2, 1, 1500), (0, 1, 5)), ((2, 8, 2, 3, 1500), (0, 3)), ((2, 4, 2, 200, 333), (0, 1, 2)),
                                              ((1, 2, 1, 70, 70), (0,)), ((1, 40, 1, 1, 40), (0,)), ((1, 136, 8, 129, 140), (0,))):
        q, k, v = inputs(2500 + D + Dv + Sq, B, Hq, Hkv, Sq, Skv, D, Dv, dtype)
        lens = np.array([Skv, max(Skv // 3, 1)][:B], np.int32)
        ref = oracle_full(q, k, v, G=Hq // Hkv, causal=True, kv_lens=lens)
        for splits in split_list:
            say("head dimension above 128: %s D=%d Dv=%d %r splits=%d" % (dtypes.NAMES[dtype], D, Dv, (B, Hq, Hkv, Sq, Skv), splits))
            got, lse, info = host.sdpa(q, k, v, dtype, causal=True, kv_lens=lens, num_splits=splits, impl=capi.IMPL_SPLITKV_MFMA,
                                       return_info=True, return_lse=True)
            check(got, ref, tol, "D=%d Dv=%d Sq=%d splits=%d->%d" % (D, Dv, Sq, splits, info["splits"]))
        got, lse, info = host.sdpa(q, k, v, dtype, causal=True, kv_lens=lens, return_info=True, return_lse=True)
        # (16-bit: the prefill kernel for 256 once its 128-row workgroups cover more than half the compute units)
        cus, wgs, chunks = capi.device_info(0).compute_units, B * Hq * ((Sq + 127) // 128), B * Hkv * ((Hq // Hkv * Sq + 31) // 32)
        split_ahead = (wgs * 4 <= cus and (Skv >= 2048 or chunks * 2 <= cus or chunks % cus == 0)) or (wgs * 2 <= cus and chunks % cus == 0)
        prefill_256 = Sq > 64 and dtype != capi.F32 and not split_ahead
        assert info["impl"] == (capi.IMPL_MFMA if prefill_256 else capi.IMPL_SPLITKV_MFMA)
        check(got, ref, tol, "AUTO, D=%d Dv=%d Sq=%d" % (D, Dv, Sq))
        if Sq > 64 and dtype != capi.F32:
            got, lse_p, info = host.sdpa(q, k, v, dtype, causal=True, kv_lens=lens, impl=capi.IMPL_MFMA, return_info=True, return_lse=True)
            assert info["impl"] == capi.IMPL_MFMA
            check(got, ref, tol, "prefill kernel for 256, D=%d Dv=%d Sq=%d" % (D, Dv, Sq))
            fin = np.isfinite(lse)
            assert np.array_equal(fin, np.isfinite(lse_p)) and np.max(np.abs(lse[fin] - lse_p[fin])) < 2e-2
        _, lse_g = host.sdpa(q, k, v, dtype, causal=True, kv_lens=lens, impl=capi.IMPL_GENERIC, return_lse=True)
        fin = np.isfinite(lse_g)
        assert np.array_equal(fin, np.isfinite(lse)) and np.max(np.abs(lse[fin] - lse_g[fin])) < (2e-5 if dtype == capi.F32 else 2e-2)


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16], ids=lambda x: dtypes.NAMES[x])
@pytest.mark.parametrize("dims", [(256, 256), (192, 128)], ids=lambda x: "D%d_Dv%d" % x)
def test_head_dimensions_above_128_with_a_dense_mask(gpu, dtype, dims):
    """The prefill kernel for 256 with a dense additive mask: a sliding window given as a [1, 1, Sq, Skv] tensor (tiles before
    the window are skipped by the mask's block flags), random values with hidden blocks per batch entry on top of the causal
    flag, a decode-like launch with a mask; a mask whose rows are not 8-byte aligned falls to the generic kernel."""
    D, Dv = dims
    tol = TOL[dtype]
    B, Hq, Hkv, Sq, Skv = 2, 4, 2, 300, 420
    q, k, v = inputs(2600 + D, B, Hq, Hkv, Sq, Skv, D, Dv, dtype)
    i, j = np.arange(Sq)[:, None], np.arange(Skv)[None, :]
    window = np.where((j <= i + Skv - Sq) & (j > i + Skv - Sq - 100), 0.0, -np.inf).astype(np.float32)[None, None]
    got, info = host.sdpa(q, k, v, dtype, mask=window, return_info=True)
    assert info["impl"] == capi.IMPL_MFMA
    check(got, oracle_full(q, k, v, G=2, mask=window), tol, "sliding window as a tensor, D=%d" % D)
    r = rng(7)
    m = (r.standard_normal((B, 1, Sq, Skv)) * 0.5).astype(np.float32)
    m[0, :, 64:200, 32:160] = -np.inf
    m[1, :, :, 300:] = -np.inf
    m = dtypes.round_to(m, dtype)
    got, lse, info = host.sdpa(q, k, v, dtype, mask=m, causal=True, return_info=True, return_lse=True)
    assert info["impl"] == capi.IMPL_MFMA
    full = np.broadcast_to(m, (B, Hq, Sq, Skv)) + np.triu(np.full((Sq, Skv), -np.inf, np.float32), 1 + Skv - Sq)
    check(got, oracle_full(q, k, v, G=2, mask=full), tol, "random mask with hidden blocks + causal, D=%d" % D)
    _, lse_g = host.sdpa(q, k, v, dtype, mask=m, causal=True, impl=capi.IMPL_GENERIC, return_lse=True)
    assert np.max(np.abs(lse - lse_g)) < 2e-2
    # decode-like: 3 positions over the cache with a mask
    q3 = q[:, :, :3]
    got, info = host.sdpa(q3, k, v, dtype, mask=m[:, :, :3], return_info=True)
    assert info["impl"] == capi.IMPL_MFMA          # (420 keys: not a multiple of 8, so not for the split-KV kernel's mask copies)
    check(got, oracle_full(q3, k, v, G=2, mask=m[:, :, :3]), tol, "decode-like with a mask, D=%d" % D)
    got, info = host.sdpa(q3, k[:, :, :416], v[:, :, :416], dtype, mask=m[:, :, :3, :416], return_info=True)
    assert info["impl"] == capi.IMPL_SPLITKV_MFMA          # (416 keys: up to 64 positions go to the split-KV kernel with their mask)
    check(got, oracle_full(q3, k[:, :, :416], v[:, :, :416], G=2, mask=m[:, :, :3, :416]), tol, "decode-like with a mask on the split-KV kernel, D=%d" % D)
    # 418 keys: rows of the mask 836 bytes apart
    got, info = host.sdpa(q, k[:, :, :418], v[:, :, :418], dtype, mask=m[..., :418], return_info=True)
    assert info["impl"] == capi.IMPL_GENERIC
    check(got, oracle_full(q, k[:, :, :418], v[:, :, :418], G=2, mask=m[..., :418]), tol, "mask rows not 8-byte aligned: generic")


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16], ids=lambda x: dtypes.NAMES[x])
@pytest.mark.parametrize("skv", [417, 418, 419, 33], ids=lambda x: "skv%d" % x)
def test_head_dimensions_above_128_key_bias_on_the_last_keys(gpu, dtype, skv):
    """A key bias [1, 1, 1, Skv] (every stride but the key's is 0, so the prefill kernel for 256 takes it) with Skv not a
    multiple of 4: the last Skv % 4 keys carry -inf and a large bias, which the kernel must add like any other key's."""
    D = Dv = 256
    B, Hq, Hkv, Sq = 2, 4, 2, 200
    q, k, v = inputs(2700 + skv, B, Hq, Hkv, Sq, skv, D, Dv, dtype)
    bias = (rng(8).standard_normal((1, 1, 1, skv)) * 0.5).astype(np.float32)
    bias[..., skv - 1] = -np.inf
    if skv % 4 >= 2:
        bias[..., skv - 2] = 6.0
    if skv % 4 == 3:
        bias[..., skv - 3] = -np.inf
    bias = dtypes.round_to(bias, dtype)
    say("key bias on the last keys: %s Skv=%d" % (dtypes.NAMES[dtype], skv))
    got, info = host.sdpa(q, k, v, dtype, mask=bias, return_info=True)
    assert info["impl"] == capi.IMPL_MFMA
    ref = oracle_full(q, k, v, G=2, mask=np.broadcast_to(bias, (1, 1, Sq, skv)))
    check(got, ref, TOL[dtype], "key bias with values on the last %d keys, D=256" % (skv % 4))
    # the same with the rows of a [B, 1, Sq, Skv] mask padded to a pitch of whole 8-byte groups
    pitch = (skv + 3) // 4 * 4 + 4
    mp = (rng(9).standard_normal((B, 1, Sq, skv)) * 0.5).astype(np.float32)
    mp[..., skv - 1] = -np.inf
    mp[0, 0, 5, skv - 1] = 3.0
    mp = dtypes.round_to(mp, dtype)
    got, info = host.sdpa(q, k, v, dtype, mask=mp, mask_row_pitch=pitch, return_info=True)
    assert info["impl"] == capi.IMPL_MFMA
    check(got, oracle_full(q, k, v, G=2, mask=mp), TOL[dtype], "mask rows at a padded pitch, D=256")


def test_head_dimensions_outside_the_matrix_core_kernels(gpu):
    """Rows that are not whole 16-byte vectors stay on the generic kernel."""
    for dtype, D in ((capi.BF16, 20), (capi.F32, 6), (capi.BF16, 132), (capi.F32, 134)):
        q, k, v = inputs(2400 + D, 1, 2, 2, 40, 70, D, D, dtype)
        got, info = host.sdpa(q, k, v, dtype, causal=True, return_info=True)
        assert info["impl"] == capi.IMPL_GENERIC
        check(got, oracle_full(q, k, v, causal=True), TOL[dtype], "generic D=%d" % D)


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16, capi.F32], ids=lambda x: dtypes.NAMES[x])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, D
    (2, 8, 2, 1, 1500, 128),          # grouped-query decode, 4 rows per KV head
    (3, 4, 4, 1, 700, 64),            # one row per KV head
    (1, 16, 2, 1, 2049, 128),         # 8 rows, a ragged last tile
    (2, 4, 2, 3, 900, 64),            # 6 rows: a short causal run
])
def test_decode_with_a_dense_additive_mask(gpu, dtype, shape):
    """Decode shapes with a mask tensor - an additive position bias per head ([1, Hq, 1, Skv]) and a [B, 1, Sq, Skv] mask with
    hidden stretches, on top of key counts - go through the vector-ALU split-KV kernel (up to 8 rows per KV head), which
    adds the mask's values to the scaled scores: against the oracle, split counts chosen and forced."""
    B, Hq, Hkv, Sq, Skv, D = shape
    q, k, v = inputs(2700 + sum(shape), B, Hq, Hkv, Sq, Skv, D, D, dtype)
    bias = (-0.02 * np.arange(Skv)[::-1].astype(np.float32))[None, None, None, :] * (1.0 + np.arange(Hq, dtype=np.float32))[None, :, None, None]
    bias = dtypes.round_to(np.broadcast_to(bias, (1, Hq, Sq, Skv)).copy(), dtype)
    r = rng(17)
    holes = (r.standard_normal((B, 1, Sq, Skv)) * 0.3).astype(np.float32)
    holes[:, :, :, 100:400] = -np.inf
    holes[0, :, :, Skv - 50:] = -np.inf
    holes = dtypes.round_to(holes, dtype)
    lens = np.array([Skv - 7 * b for b in range(B)], np.int32)
    for name, m in (("bias per head", bias), ("holes per batch entry", holes)):
        full = np.broadcast_to(m, (B, Hq, Sq, Skv)) + np.where(np.arange(Skv)[None, :] < lens[:, None], 0.0, -np.inf).astype(np.float32)[:, None, None, :]
        ref = oracle_full(q, k, v, G=Hq // Hkv, mask=full)
        for splits in (0, 1, 5):
            say("decode with a mask: %s %r %s splits=%d" % (dtypes.NAMES[dtype], shape, name, splits))
            got, info = host.sdpa(q, k, v, dtype, mask=m, kv_lens=lens, num_splits=splits, impl=capi.IMPL_SPLITKV, return_info=True)
            assert info["impl"] == capi.IMPL_SPLITKV
            check(got, ref, TOL[dtype], "decode with a mask (%s), splits=%d->%d" % (name, splits, info["splits"]))
            got, info = host.sdpa(q, k, v, dtype, mask=m, kv_lens=lens, num_splits=splits, return_info=True)
            # (AUTO: f32 and key counts that are not multiples of 4 stay on the vector-ALU kernel, 16-bit launches follow the
            # thresholds of launches without a mask)
            assert info["impl"] in (capi.IMPL_SPLITKV, capi.IMPL_SPLITKV_MFMA)
            if dtype == capi.F32 or Skv % 8:
                assert info["impl"] == capi.IMPL_SPLITKV
            check(got, ref, TOL[dtype], "decode with a mask (%s), AUTO, splits=%d->%d" % (name, splits, info["splits"]))


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16], ids=lambda x: dtypes.NAMES[x])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, D
    (2, 8, 2, 1, 1496, 128),          # grouped-query decode, 4 rows per KV head
    (1, 16, 2, 1, 2056, 128),         # 8 rows, a ragged last block
    (2, 4, 2, 3, 904, 64),            # 6 rows: a short causal run; blocks of 64 keys
    (1, 48, 1, 1, 1000, 128),         # 48 rows: two blocks of rows per workgroup
    (2, 8, 2, 5, 640, 64),            # 20 rows, causal among themselves
    (1, 8, 2, 1, 1200, 256),          # the 256 instance
    (3, 4, 4, 1, 4104, 128),          # one row per KV head
    (2, 8, 2, 1, 40, 128),            # a cache shorter than one round of blocks
], ids=lambda x: "x".join(map(str, x)))
def test_decode_with_a_dense_additive_mask_on_the_matrix_cores(gpu, dtype, shape):
    """The matrix-core split-KV kernel with a mask tensor: a position bias per head ([1, Hq, 1, Skv]), a [B, 1, Sq, Skv] mask
    with hidden stretches and a full [B, Hq, Sq, Skv] one, with key counts and (where there are several positions) the causal
    flag on top - against the oracle, for the split counts the planner chooses and forced ones (a split that ends inside a
    block, splits whose keys the mask hides entirely), and against the vector-ALU kernel where that takes the launch."""
    B, Hq, Hkv, Sq, Skv, D = shape
    q, k, v = inputs(2900 + sum(shape), B, Hq, Hkv, Sq, Skv, D, D, dtype)
    bias = (-0.02 * np.arange(Skv)[::-1].astype(np.float32))[None, None, None, :] * (1.0 + np.arange(Hq, dtype=np.float32))[None, :, None, None]
    bias = dtypes.round_to(np.ascontiguousarray(np.broadcast_to(bias, (1, Hq, 1, Skv))), dtype)
    r = rng(18)
    holes = (r.standard_normal((B, 1, Sq, Skv)) * 0.3).astype(np.float32)
    holes[:, :, :, 100:400] = -np.inf
    holes[0, :, :, Skv - 50:] = -np.inf
    holes = dtypes.round_to(holes, dtype)
    full_m = dtypes.round_to((r.standard_normal((B, Hq, Sq, Skv)) * 0.5).astype(np.float32), dtype)
    full_m[:, 0, :, :] = -np.inf                       # one head sees nothing: NaN rows, as the reference gives
    lens = np.array([Skv - 7 * b for b in range(B)], np.int32)
    causal = Sq > 1
    tri = np.triu(np.full((Sq, Skv), -np.inf, np.float32), 1 + Skv - Sq) if causal else np.zeros((Sq, Skv), np.float32)
    for name, m in (("bias per head", bias), ("holes per batch entry", holes), ("full mask", full_m)):
        full = np.broadcast_to(m, (B, Hq, Sq, Skv)) + tri + np.where(np.arange(Skv)[None, :] < lens[:, None], 0.0, -np.inf).astype(np.float32)[:, None, None, :]
        ref = oracle_full(q, k, v, G=Hq // Hkv, mask=full)
        for splits in (0, 1, 3, 7):
            say("matrix-core decode with a mask: %s %r %s splits=%d" % (dtypes.NAMES[dtype], shape, name, splits))
            got, info = host.sdpa(q, k, v, dtype, mask=m, kv_lens=lens, causal=causal, num_splits=splits, impl=capi.IMPL_SPLITKV_MFMA, return_info=True)
            assert info["impl"] == capi.IMPL_SPLITKV_MFMA
            check(got, ref, TOL[dtype], "matrix-core decode with a mask (%s), splits=%d->%d" % (name, splits, info["splits"]))
    # a mask it cannot copy eight keys at a time is refused by name and goes elsewhere under AUTO
    with pytest.raises(capi.RocmError):
        host.sdpa(q, k[:, :, :Skv - 4], v[:, :, :Skv - 4], dtype, mask=bias[..., :Skv - 4], impl=capi.IMPL_SPLITKV_MFMA)
    got, info = host.sdpa(q, k[:, :, :Skv - 4], v[:, :, :Skv - 4], dtype, mask=bias[..., :Skv - 4], return_info=True)
    assert info["impl"] != capi.IMPL_SPLITKV_MFMA


def test_decode_splitkv_matrix_cores_lengths_strides_scale(gpu):
    """Key counts per batch entry (one of them 0: NaN rows, as the reference), a negative scale (the scale is applied to
    the f32 scores, so its sign does not matter to this kernel), and AUTO's choice for grouped-query decode."""
    B, Hq, Hkv, Skv, D = 4, 16, 4, 1100, 128
    q, k, v = inputs(733, B, Hq, Hkv, 1, Skv, D, D, capi.BF16)
    lens = np.array([1100, 64, 0, 257], np.int32)
    for splits in (0, 1, 5):
        got, info = host.sdpa(q, k, v, capi.BF16, kv_lens=lens, num_splits=splits, impl=capi.IMPL_SPLITKV_MFMA, return_info=True)
        ref = oracle_full(q, k, v, G=4, kv_lens=lens)
        assert np.isnan(ref[2]).all()
        check(got, ref, 2e-2, "matrix-core split-KV kv_lens incl. empty, splits=%d" % splits)
    got = host.sdpa(q, k, v, capi.BF16, scale=-0.07, impl=capi.IMPL_SPLITKV_MFMA)
    check(got, oracle_full(q, k, v, G=4, scale=-0.07), 2e-2, "matrix-core split-KV negative scale")
    got, info = host.sdpa(q, k, v, capi.BF16, return_info=True)
    assert info["impl"] == capi.IMPL_SPLITKV_MFMA           # 4 rows per KV head, 16-bit, D = 128: AUTO's choice
    check(got, oracle_full(q, k, v, G=4), 2e-2, "AUTO grouped-query decode")
    _, info = host.sdpa(q[:, :4], k, v, capi.BF16, return_info=True)
    assert info["impl"] == capi.IMPL_SPLITKV                # one row per KV head stays on the vector-ALU kernel


@pytest.mark.parametrize("impl", [capi.IMPL_SPLITKV_MFMA, capi.IMPL_SPLITKV], ids=["matrix_cores", "vector_alu"])
def test_decode_over_a_token_major_cache(gpu, impl):
    """Cache, queries and output stored [B, S, H, D] (token-major, as serving stacks keep them) and handed over as
    [B, H, S, D] views by strides alone: both split-KV kernels read rows 'Hkv * D' elements apart in place."""
    B, Hq, Hkv, Sq, Skv, D = 2, 8, 2, 2, 1111, 128
    dt = capi.BF16
    q, k, v = inputs(811, B, Hq, Hkv, Sq, Skv, D, D, dt)
    ref = oracle_full(q, k, v, G=Hq // Hkv, causal=True)
    tq, tk, tv = (host.DeviceTensor.from_f32(np.ascontiguousarray(x.transpose(0, 2, 1, 3)), dt) for x in (q, k, v))
    to = host.DeviceTensor((B, Sq, Hq, D), dt)

    class View:                                   # logical [B, H, S, D] over the stored [B, S, H, D]
        def __init__(self, t, H, S):
            self.shape, self.dtype, self.dev, self.ptr = (B, H, S, D), t.dtype, t.dev, t.ptr
    d = host.make_desc(View(tq, Hq, Sq), View(tk, Hkv, Skv), View(tv, Hkv, Skv), View(to, Hq, Sq), causal=True, impl=impl, num_splits=3)
    for name, H, S in (("q_stride", Hq, Sq), ("k_stride", Hkv, Skv), ("v_stride", Hkv, Skv), ("o_stride", Hq, Sq)):
        st = getattr(d, name)
        st[0], st[1], st[2] = S * H * D, D, H * D
    nbytes, splits, chosen = capi.sdpa_workspace(d)
    assert chosen == impl and splits == 3
    ws = capi.DeviceBuffer(nbytes)
    d.workspace, d.workspace_bytes = ws.ptr, ws.nbytes
    capi.sdpa_fwd(d)
    capi.sync()
    got = to.to_f32().transpose(0, 2, 1, 3)
    check(got, ref, TOL[dt], "token-major cache, impl %d" % impl)
    for t in (tq, tk, tv, to):
        t.buf.free()
    ws.free()


def test_decode_lengths_and_prefill_consistency(gpu):
    B, H, Skv, D = 3, 4, 2048, 128
    q, k, v = inputs(41, B, H, H, 1, Skv, D, D, capi.BF16)
    lens = np.array([2048, 5, 0], np.int32)
    got = host.sdpa(q, k, v, capi.BF16, kv_lens=lens, num_splits=4)
    ref = oracle_full(q, k, v, kv_lens=lens)
    assert np.isnan(ref[2]).all()
    check(got, ref, 2e-2, "decode kv_lens incl. empty")
    # decode output == last row of causal prefill over the same cache
    qf, kf, vf = inputs(42, 1, 2, 2, 512, 512, 128, 128, capi.BF16)
    full = host.sdpa(qf, kf, vf, capi.BF16, causal=True, impl=capi.IMPL_MFMA)
    last = host.sdpa(qf[:, :, -1:], kf, vf, capi.BF16, causal=True)
    check(last, full[:, :, -1:], 8e-3, "decode == last row of causal prefill")


@pytest.mark.parametrize("impl, dtype, sq", [
    (capi.IMPL_GENERIC, capi.F32, 70), (capi.IMPL_GENERIC, capi.BF16, 70), (capi.IMPL_MFMA, capi.BF16, 200),
    (capi.IMPL_MFMA, capi.F16, 200), (capi.IMPL_SPLITKV, capi.BF16, 1), (capi.IMPL_SPLITKV, capi.F32, 2),
    (capi.IMPL_SPLITKV_MFMA, capi.BF16, 3), (capi.IMPL_SPLITKV_MFMA, capi.F16, 1)],
    ids=["generic_f32", "generic_bf16", "mfma_bf16", "mfma_f16", "splitkv_bf16", "splitkv_f32", "splitkv_mfma_bf16", "splitkv_mfma_f16"])
def test_rows_beyond_the_key_count_are_never_read(gpu, impl, dtype, sq):
    """A preallocated cache holds whatever the allocator left behind its valid rows.  With NaN and infinity bit patterns
    in every key and value row at and beyond kv_lens[b], each kernel gives the bytes it gives over a zeroed tail, and
    those agree with the oracle on the truncated operands."""
    B, Hq, Hkv, Skv, D = 3, 4, 2, 333, 128
    lens = np.array([333, 97, 1], np.int32)
    q, k, v = inputs(SEED0 + 71, B, Hq, Hkv, sq, Skv, D, D, dtype)
    k_bad, v_bad = k.copy(), v.copy()
    junk = np.array([np.nan, np.inf, -np.inf, np.nan], np.float32)
    for b in range(B):
        n = Skv - lens[b]
        if n:
            k[b, :, lens[b]:], v[b, :, lens[b]:] = 0.0, 0.0
            fill = np.resize(junk, n * D).reshape(n, D)
            k_bad[b, :, lens[b]:], v_bad[b, :, lens[b]:] = fill, fill[::-1]
    say("junk beyond kv_lens: impl %d dtype %d" % (impl, dtype))
    kw = dict(causal=False, kv_lens=lens, impl=impl, num_splits=3 if impl in (capi.IMPL_SPLITKV, capi.IMPL_SPLITKV_MFMA) else 0)
    clean, info = host.sdpa(q, k, v, dtype, return_info=True, **kw)
    assert info["impl"] == impl
    dirty = host.sdpa(q, k_bad, v_bad, dtype, **kw)
    assert np.isfinite(dirty).all()
    assert np.array_equal(dirty, clean)
    check(dirty, oracle_full(q, k, v, G=Hq // Hkv, kv_lens=lens), TOL[dtype], "junk tail")


@pytest.mark.parametrize("impl, sq", [(capi.IMPL_MFMA, 96), (capi.IMPL_SPLITKV, 2), (capi.IMPL_GENERIC, 40),
                                      (capi.IMPL_SPLITKV_MFMA, 6)],
                         ids=["mfma", "splitkv", "generic", "splitkv_mfma"])
@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16])
def test_large_logits(gpu, dtype, impl, sq):
    """Logits of magnitude 50 with many keys within a few units of each row's maximum, and query rows whose elements are
    all equal - so that whatever rounding a kernel applies to a query element (the matrix-core kernels fold
    scale * log2(e) into Q and round it back to the storage type) hits every element of the row the same way and shows
    up as a relative error of the whole logit row instead of averaging out.  Same absolute bar as everywhere."""
    B, H, Skv, D = 2, 2, 320, 128
    r = rng(SEED0 + 90)
    x = r.choice(np.array([1.7265625, 1.8359375, 1.9140625, 2.0546875, 2.1328125], np.float32), size=(B, H, sq, 1))
    q = dtypes.round_to(np.broadcast_to(x * r.choice([-1.0, 1.0], size=(B, H, sq, 1)).astype(np.float32), (B, H, sq, D)).copy(), dtype)
    c = r.uniform(-2.2, 2.2, size=(B, H, Skv, 1)).astype(np.float32)
    k = dtypes.round_to(c + 0.05 * r.standard_normal((B, H, Skv, D), dtype=np.float32), dtype)
    v = dtypes.round_to(r.standard_normal((B, H, Skv, D), dtype=np.float32), dtype)
    logits = np.einsum("bhid,bhjd->bhij", q, k) / np.sqrt(np.float32(D))
    top = np.sort(logits, axis=-1)[..., -8:]
    say("large logits: impl %d dtype %d, max |logit| %.1f, 8th-largest within %.2f of the row maximum (median)"
        % (impl, dtype, np.abs(logits).max(), np.median(top[..., -1] - top[..., 0])))
    assert np.abs(logits).max() > 45
    got, info = host.sdpa(q, k, v, dtype, impl=impl, return_info=True, num_splits=2 if impl in (capi.IMPL_SPLITKV, capi.IMPL_SPLITKV_MFMA) else 0)
    assert info["impl"] == impl
    check(got, oracle_full(q, k, v), TOL[dtype], "large logits")


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16])
@pytest.mark.parametrize("shape", [
    # B, Hq, Hkv, Sq, Skv, causal, kv_lens, q_lens
    (1, 2, 2, 640, 640, True, None, None),
    (1, 2, 1, 700, 700, False, None, None),                       # rows and keys not multiples of the blocks
    (2, 4, 2, 513, 900, True, [900, 311], None),                  # Sq < Skv: causal alignment; ragged keys
    (2, 2, 2, 900, 300, True, None, None),                        # Sq > Skv: rows without keys
    (3, 2, 2, 768, 768, True, [768, 200, 0], [768, 200, 0]),      # a padded batch: padding rows, an empty sequence
    (1, 1, 1, 255, 257, False, [129], None),
], ids=["square", "ragged_edges", "gqa_lens", "rows_without_keys", "padded_batch", "short"])
def test_256_row_workgroups(gpu, dtype, shape, monkeypatch):
    """The 16-bit prefill kernel runs with 128 or 256 query rows per workgroup (the launcher picks by the size of the
    problem; INCIN_ROCM_PREFILL_BLOCK_ROWS forces one).  A row's arithmetic does not depend on which: both forms must agree
    bit for bit on every valid row, normalisers included, and with the oracle."""
    B, Hq, Hkv, Sq, Skv, causal, kv_lens, q_lens = shape
    q, k, v = inputs(700 + Sq + Skv, B, Hq, Hkv, Sq, Skv, 128, 128, dtype)
    kl = None if kv_lens is None else np.asarray(kv_lens, np.int32)
    qlens = None if q_lens is None else np.asarray(q_lens, np.int32)
    outs = {}
    for rows in ("128", "256"):
        monkeypatch.setenv("INCIN_ROCM_PREFILL_BLOCK_ROWS", rows)
        outs[rows] = host.sdpa(q, k, v, dtype, causal=causal, kv_lens=kl, q_lens=qlens, impl=capi.IMPL_MFMA, return_lse=True)
    monkeypatch.delenv("INCIN_ROCM_PREFILL_BLOCK_ROWS")
    (o128, l128), (o256, l256) = outs["128"], outs["256"]
    valid = np.ones((B, Hq, Sq), bool)
    if qlens is not None:
        valid &= np.arange(Sq)[None, None, :] < qlens[:, None, None]
    assert np.array_equal(o128[valid], o256[valid], equal_nan=True)
    assert np.array_equal(l128[valid], l256[valid], equal_nan=True)
    ref = oracle_full(q, k, v, G=Hq // Hkv, causal=causal, kv_lens=kl)
    got = np.where(valid[..., None], o256, ref)
    check(got, ref, TOL[dtype], "256-row workgroups %r" % (shape,))


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16], ids=lambda x: dtypes.NAMES[x])
@pytest.mark.parametrize("dims", [(96, 96), (80, 96), (96, 72), (72, 40)], ids=lambda x: "D%d_Dv%d" % x)
@pytest.mark.parametrize("rows", ["128", "256"])
def test_head_dimensions_up_to_96_in_the_128_layout(gpu, dtype, dims, rows, monkeypatch):
    """Head dimensions between 65 and 96 (D and Dv both) run an instance of the 16-bit prefill kernel that keeps the 128-column
    layout of a tile in LDS but leaves the last quarter out of both matrix products: 6 of 8 k-steps, 3 of 4 output blocks.
    Its pipelined loop deals the softmax over the k-steps differently, so it gets what the full instance gets: enough
    tiles for the loop to run in both workgroup forms, ragged edges, key counts, grouped queries, and the keys far above
    the reference that make the loop back out of a tile."""
    D, Dv = dims
    monkeypatch.setenv("INCIN_ROCM_PREFILL_BLOCK_ROWS", rows)
    for B, Hq, Hkv, Sq, Skv, causal, kv_lens in ((1, 2, 2, 640, 640, True, None), (1, 2, 1, 700, 900, False, None),
                                                  (2, 4, 2, 513, 1100, True, [1100, 311])):
        say("head dimension %d/%d, %s rows: %s" % (D, Dv, rows, (B, Hq, Hkv, Sq, Skv, causal, kv_lens)))
        q, k, v = inputs(2900 + D + Dv + Sq, B, Hq, Hkv, Sq, Skv, D, Dv, dtype)
        kl = None if kv_lens is None else np.asarray(kv_lens, np.int32)
        got, lse, info = host.sdpa(q, k, v, dtype, causal=causal, kv_lens=kl, impl=capi.IMPL_MFMA, return_info=True, return_lse=True)
        assert info["impl"] == capi.IMPL_MFMA and got.shape[-1] == Dv
        check(got, oracle_full(q, k, v, G=Hq // Hkv, causal=causal, kv_lens=kl), TOL[dtype], "D=%d Dv=%d %s rows" % (D, Dv, rows))
        _, lse_g = host.sdpa(q, k, v, dtype, causal=causal, kv_lens=kl, impl=capi.IMPL_GENERIC, return_lse=True)
        assert np.max(np.abs(lse - lse_g)) < 2e-2
    # keys 60 to 130 logit units above what a row saw before (as in the test below), identical within a class
    B, H, S = 1, 2, 640
    r = rng(SEED0 + 94)
    a = r.choice(np.array([1.0, -1.0, 0.5], np.float32), size=(B, H, S, 1))
    q = np.broadcast_to(a, (B, H, S, D)).copy()
    b = np.full((B, H, S, 1), -4.0, np.float32)
    b[:, :, [70, 200, 201, 207, 231, 250]] = 2.0
    b[:, :, [400, 401, 437]] = 8.0
    b[:, 1, 100] = 8.0
    k = np.broadcast_to(b, (B, H, S, D)).copy()
    v = dtypes.round_to(r.standard_normal((B, H, S, Dv), dtype=np.float32), dtype)
    for causal in (False, True):
        got = host.sdpa(q, k, v, dtype, causal=causal, impl=capi.IMPL_MFMA, scale=1.0 / np.sqrt(128.0))
        logit = a * np.swapaxes(b, 2, 3)
        if causal:
            logit = np.where(np.tril(np.ones((S, S), bool)), logit, -np.inf)
        top = logit == logit.max(axis=-1, keepdims=True)
        mean = np.einsum("bhij,bhjd->bhid", top.astype(np.float64), v.astype(np.float64)) / top.sum(axis=-1, keepdims=True)
        check(got, mean.astype(np.float32), TOL[dtype], "scores far above the first tiles, D=%d Dv=%d" % (D, Dv))


@pytest.mark.parametrize("causal", [False, True, "tensor"], ids=["full", "causal", "causal_as_tensor"])
@pytest.mark.parametrize("impl", [capi.IMPL_MFMA], ids=["mfma"])
@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16])
@pytest.mark.parametrize("rows", ["128", "256"])
def test_scores_far_above_the_first_tiles(gpu, dtype, impl, causal, rows, monkeypatch):
    """Keys whose logits lie 60 to 130 units above everything a row has seen before, in the second, the fourth and the
    seventh key tile: the reference maximum a kernel carries from earlier tiles is useless there.  The 16-bit prefill
    kernel takes no maxima in its pipelined loop for bf16 (it watches one bit of the probabilities instead) and has to
    notice, rescale and take the probabilities of that tile again; rows of the opposite sign see the same keys fall
    130 units below their maximum and must not notice at all, and rows of half the magnitude stay under the trigger
    while sharing a wavefront with rows that pull it.  Keys of one class are identical, so every row's answer is a
    plain mean of V rows and the rounding of the pre-scaled queries cannot matter."""
    if rows == "256" and (impl != capi.IMPL_MFMA or causal == "tensor"):
        pytest.skip("256-row workgroups: the 32-row kernel without a dense mask")
    monkeypatch.setenv("INCIN_ROCM_PREFILL_BLOCK_ROWS", rows)
    B, H, S, D = 1, 2, 640, 128
    r = rng(SEED0 + 93)
    a = r.choice(np.array([1.0, -1.0, 0.5], np.float32), size=(B, H, S, 1))
    q = np.broadcast_to(a, (B, H, S, D)).copy()
    b = np.full((B, H, S, 1), -4.0, np.float32)
    b[:, :, [70, 200, 201, 207, 231, 250]] = 2.0
    b[:, :, [400, 401, 437]] = 8.0
    b[:, 1, 100] = 8.0                                       # head 1: the largest class already in the second tile
    k = np.broadcast_to(b, (B, H, S, D)).copy()
    v = dtypes.round_to(r.standard_normal((B, H, S, D), dtype=np.float32), dtype)
    if causal == "tensor":
        # the causal mask the way the reference's operator takes it: the dense-mask instance of the kernel, whose
        # mask-free stretch of tiles runs the same bit check
        mask = O.causal_additive_mask(S, S).reshape(1, 1, S, S)
        got, info = host.sdpa(q, k, v, dtype, mask=mask, impl=impl, return_info=True)
        causal = True
    else:
        got, info = host.sdpa(q, k, v, dtype, causal=causal, impl=impl, return_info=True)
    assert info["impl"] == impl
    ref = oracle_full(q, k, v, causal=causal)
    check(got, ref, TOL[dtype], "scores far above the first tiles")
    # the closed form: mean of the V rows of the visible keys with the row's largest logit
    logit = a * np.swapaxes(b, 2, 3)                                  # [B, H, S, S] up to a positive factor
    if causal:
        logit = np.where(np.tril(np.ones((S, S), bool)), logit, -np.inf)
    top = logit == logit.max(axis=-1, keepdims=True)
    mean = np.einsum("bhij,bhjd->bhid", top.astype(np.float64), v.astype(np.float64)) / top.sum(axis=-1, keepdims=True)
    check(got, mean.astype(np.float32), TOL[dtype], "scores far above the first tiles, closed form")


def test_matrix_rate_diagnostic(gpu):
    """The matrix-instruction loop behind bench.py's matrix_rate figures: it runs, and counts its own work."""
    info = capi.device_info(0)
    sink = capi.DeviceBuffer(2048 * info.compute_units)
    src = capi.DeviceBuffer.from_numpy(np.zeros(65536, np.uint32))
    for mix in (0, 1):
        fl = capi.matrix_rate(src, sink, mix, 100)
        capi.sync()
        assert fl == info.compute_units * 8 * 100 * 4 * 32768.0
    src.free()
    sink.free()


def test_padded_head_dimensions_do_not_depend_on_what_lds_held(gpu):
    """The matrix-core kernels pad a head dimension below their instance's with zeros the copy engine writes into LDS
    (lanes whose 16 bytes lie beyond a row's data address memory no descriptor covers and deliver zeros).  Were those
    lanes to write nothing, the padding would be whatever the last kernel left in LDS - usually small numbers, so an
    ordinary parity test could pass by luck.  Fill every compute unit's LDS with NaN bit patterns (as bf16/f16 pairs,
    as f32, all ones) before each launch: results carry no NaN, match the oracle and are bit-identical to the launch
    before the fill."""
    BF, F = capi.BF16, capi.F32
    cases = [  # dtype, D, Dv, Hq, Sq, Skv, causal, impl asked, impl run
        (BF, 96, 96, 4, 200, 333, True, capi.IMPL_AUTO, capi.IMPL_MFMA),                 # prefill, 128 instance
        (capi.F16, 40, 72, 4, 200, 333, True, capi.IMPL_AUTO, capi.IMPL_MFMA),           # prefill, D and Dv in different instances' reach
        (BF, 40, 72, 4, 1, 1500, False, capi.IMPL_AUTO, capi.IMPL_SPLITKV_MFMA),         # decode
        (BF, 192, 128, 4, 200, 333, True, capi.IMPL_MFMA, capi.IMPL_MFMA),               # prefill kernel for 256
        (BF, 192, 128, 4, 200, 333, True, capi.IMPL_AUTO, capi.IMPL_SPLITKV_MFMA),       # a launch this small: split-KV, 256 instance
        (BF, 160, 160, 8, 1, 1500, False, capi.IMPL_AUTO, capi.IMPL_SPLITKV_MFMA),       # decode, 256 instance
        (F, 20, 36, 4, 200, 333, True, capi.IMPL_AUTO, capi.IMPL_SPLITKV_MFMA),          # f32: a small prefill launch
        (F, 20, 36, 4, 200, 333, True, capi.IMPL_MFMA, capi.IMPL_MFMA),                  # f32 prefill kernel
        (F, 100, 100, 8, 1, 1500, False, capi.IMPL_AUTO, capi.IMPL_SPLITKV_MFMA),        # f32 decode
    ]
    sink = capi.DeviceBuffer.from_numpy(np.full(4, 7, np.uint32))
    for dtype, D, Dv, Hq, Sq, Skv, causal, impl, impl_run in cases:
        q, k, v = inputs(2700 + D + Dv, 2, Hq, 2, Sq, Skv, D, Dv, dtype)
        ref = oracle_full(q, k, v, G=Hq // 2, causal=causal)
        first, info = host.sdpa(q, k, v, dtype, causal=causal, impl=impl, return_info=True)
        assert info["impl"] == impl_run
        for pattern in (0x7fc07fc0, 0x7e007e00, 0x7fc00000, 0xffffffff):
            say("LDS filled with %08x: %s D=%d Dv=%d Sq=%d impl %d" % (pattern, dtypes.NAMES[dtype], D, Dv, Sq, impl_run))
            capi.lds_fill(pattern, sink)
            got = host.sdpa(q, k, v, dtype, causal=causal, impl=impl)
            assert not np.isnan(got).any(), "NaN after filling LDS with %08x, D=%d Dv=%d" % (pattern, D, Dv)
            check(got, ref, TOL[dtype], "after filling LDS with %08x, D=%d Dv=%d" % (pattern, D, Dv))
            assert np.array_equal(got, first)
    capi.sync()
    assert np.array_equal(sink.to_numpy(np.uint32, (4,)), np.full(4, 7, np.uint32))
    sink.free()


def test_read_rate_diagnostic(gpu):
    """The read-only kernel runs, writes nothing (its sink keeps what it held) and takes about the time the memory system
    needs for the bytes (between 2 and 8 TB/s: a sanity range, the figure itself is bench.py's business)."""
    nbytes = 1 << 30
    src = capi.DeviceBuffer(nbytes)
    capi.check(capi.load().incin_rocm_memset(0, src.ptr, 0x11, nbytes))
    sink = capi.DeviceBuffer.from_numpy(np.full(4096, 7.0, np.float32))
    for nt in (True, False):
        capi.read_rate(src, nbytes, nt, sink)
        capi.sync()
        e0, e1 = capi.Event(), capi.Event()
        e0.record()
        for _ in range(5):
            capi.read_rate(src, nbytes, nt, sink)
        e1.record()
        capi.sync()
        rate = 5 * nbytes / (e0.elapsed_ms(e1) * 1e-3) / 1e12
        say("read rate, %s loads: %.2f TB/s" % ("non-temporal" if nt else "plain", rate))
        assert 2.0 < rate < 8.0
    assert np.array_equal(sink.to_numpy(np.float32, (4096,)), np.full(4096, 7.0, np.float32))
    src.free()
    sink.free()


def test_copy_strided_gathers_any_view(gpu):
    """incin_rocm_copy_strided against numpy's own view semantics: transposes of the last two axes and of outer axes,
    broadcast (stride 0) and reversed (negative stride) axes, offsets into a larger buffer, ranks 0 to 8, 2- and 4-byte
    elements, extents on either side of the 32 x 32 tiles."""
    import ctypes as C
    lib = capi.load()
    r = rng(SEED0 + 200)

    def gather(base, view):
        """`view` is a numpy view of the contiguous array `base`; returns its logical contents gathered on the device."""
        src = capi.DeviceBuffer.from_numpy(base)
        dst = capi.DeviceBuffer(max(view.size * view.itemsize, 1))
        off = view.__array_interface__["data"][0] - base.__array_interface__["data"][0]
        shape = (C.c_int64 * max(view.ndim, 1))(*view.shape)
        strides = (C.c_int64 * max(view.ndim, 1))(*[s // view.itemsize for s in view.strides])
        capi.check(lib.incin_rocm_copy_strided(0, dst.ptr, src.ptr + off, view.ndim, shape, strides, view.itemsize, None))
        capi.sync()
        out = dst.to_numpy(view.dtype, view.shape) if view.size else np.empty(view.shape, view.dtype)
        src.free()
        dst.free()
        return out

    for dtype in (np.float32, np.uint16):
        a = (r.standard_normal((3, 5, 70, 45)) * 100).astype(dtype)
        views = [a.transpose(0, 1, 3, 2), a.transpose(1, 0, 2, 3), a[:, :, 5:60, 3:40], a[:, ::-1], a[..., ::-1],
                 np.broadcast_to(a[:, :1], a.shape), a[1, 2], a[1, 2].T, a[0, 0, 0], a[0, 0, :, 0], a[2, 4, 33:34, 7:8],
                 a.reshape(3, 5, 7, 10, 45).transpose(0, 2, 1, 4, 3), a[:, :, :0]]
        for v in views:
            say("copy_strided: %s shape %s strides %s" % (np.dtype(dtype).name, v.shape, v.strides))
            assert np.array_equal(gather(a, v), v)
        s = np.asarray(r.integers(0, 1000), dtype=dtype)               # rank 0
        assert np.array_equal(gather(s.reshape(1), s.reshape(1)[0:1].reshape(())), s)
    b = r.standard_normal((2, 1, 2, 1, 2, 3, 2, 5)).astype(np.float32)         # rank 8, last two axes swapped
    assert np.array_equal(gather(b, b.swapaxes(-1, -2)), b.swapaxes(-1, -2))
    bad = (C.c_int64 * 9)(*[1] * 9)
    assert lib.incin_rocm_copy_strided(0, None, None, 9, bad, bad, 4, None) == capi.ESHAPE
    assert lib.incin_rocm_copy_strided(0, None, None, 1, bad, bad, 3, None) == capi.EDTYPE
