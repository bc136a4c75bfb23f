"""Randomised differential test through the C ABI: seeded random shapes, dtypes, masks, lengths, scales and kernel
choices, each compared with the CPU oracle.  The fixed sweeps of test_gpu_parity.py pick cases by hand; this one
draws combinations nobody thought of (odd extents, broadcast mask axes, lengths of 0, Sq != Skv with causal
alignment, every kernel the planner accepts for the case)."""
import sys

import numpy as np
import pytest

from incin_amd import capi, dtypes, host
from oracle import oracle as O

pytestmark = pytest.mark.gpu
TOL = {capi.F32: 1e-5, capi.F16: 2e-2, capi.BF16: 2e-2}
N_CASES = 160


def say(msg):
    print(msg, file=sys.stderr, flush=True)


def draw_case(r, head_dims=(16, 32, 64, 64, 80, 128, 128, 128, 256), other_dv=(16, 64, 128)):
    dtype = int(r.choice([capi.F32, capi.F16, capi.BF16]))
    D = int(r.choice(head_dims))
    Dv = D if r.random() < 0.8 else int(r.choice(other_dv))
    Hkv = int(r.integers(1, 4))
    G = int(r.choice([1, 1, 2, 4]))
    B = int(r.integers(1, 4))
    kind = r.choice(["prefill", "prefill", "decode", "rect"])
    if kind == "decode":
        Sq, Skv = int(r.integers(1, 5)), int(r.integers(1, 1500))
    elif kind == "rect":
        Sq, Skv = int(r.integers(1, 200)), int(r.integers(1, 400))
    else:
        Sq = Skv = int(r.integers(1, 420))
    causal = bool(r.random() < 0.5)
    lens = r.integers(0, Skv + 1, B).astype(np.int32) if r.random() < 0.4 else None
    mask = None
    if r.random() < 0.25:
        shp = [B if r.random() < 0.5 else 1, Hkv * G if r.random() < 0.5 else 1, Sq if r.random() < 0.7 else 1, Skv]
        mask = r.standard_normal(shp, dtype=np.float32)
        mask[r.random(shp) < 0.2] = -np.inf
    scale = None if r.random() < 0.6 else float(r.uniform(0.02, 0.6))
    return dict(dtype=dtype, B=B, Hkv=Hkv, G=G, Sq=Sq, Skv=Skv, D=D, Dv=Dv, causal=causal, lens=lens, mask=mask, scale=scale)


def run_case(i, c, r):
    B, Hkv, G, Sq, Skv, D, Dv, dt = c["B"], c["Hkv"], c["G"], c["Sq"], c["Skv"], c["D"], c["Dv"], c["dtype"]
    Hq = Hkv * G
    q = dtypes.round_to(r.standard_normal((B, Hq, Sq, D), dtype=np.float32), dt)
    k = dtypes.round_to(r.standard_normal((B, Hkv, Skv, D), dtype=np.float32), dt)
    v = dtypes.round_to(r.standard_normal((B, Hkv, Skv, Dv), dtype=np.float32), dt)
    mask = None if c["mask"] is None else dtypes.round_to(c["mask"], dt)
    kw = dict(scale=c["scale"], causal=c["causal"], kv_lens=c["lens"], mask=mask)
    if mask is None:
        ref = O.sdpa(q.reshape(B, Hkv, G, Sq, D), k[:, :, None], v[:, :, None], scale=c["scale"], causal=c["causal"],
                     kv_lens=None if c["lens"] is None else c["lens"].reshape(B, 1, 1))
    else:
        # the reference has one mask tensor: what the descriptor states beside it (causal, key counts) is folded into
        # an explicit [B, Hkv, G, Sq, Skv] mask for the oracle
        full = np.broadcast_to(mask, (B, Hq, Sq, Skv)).copy()
        if c["causal"]:
            full += np.triu(np.full((Sq, Skv), -np.inf, np.float32), 1 + Skv - Sq)
        if c["lens"] is not None:
            full += np.where(np.arange(Skv)[None, :] < c["lens"][:, None], 0.0, -np.inf).astype(np.float32)[:, None, None, :]
        ref = O.sdpa(q.reshape(B, Hkv, G, Sq, D), k[:, :, None], v[:, :, None], mask=full.reshape(B, Hkv, G, Sq, Skv), scale=c["scale"])
    ref = ref.reshape(B, Hq, Sq, Dv)
    sc = c["scale"] if c["scale"] is not None else 1.0 / np.sqrt(D)
    c["max_logit"] = float(np.abs(np.einsum("bhgid,bhjd->bhgij", q.reshape(B, Hkv, G, Sq, D).astype(np.float64), k.astype(np.float64))).max() * sc) if q.size and k.size else 0.0
    impls = [capi.IMPL_AUTO]
    for impl in (capi.IMPL_GENERIC, capi.IMPL_MFMA, capi.IMPL_SPLITKV, capi.IMPL_SPLITKV_MFMA):
        try:
            got, info = host.sdpa(q, k, v, dt, impl=impl, return_info=True, **kw)
        except capi.RocmError as e:
            assert e.code == 7, "case %d impl %d: %s" % (i, impl, e)       # EUNSUPPORTED: outside that kernel's domain
            continue
        impls.append(impl)
        check(i, c, impl, got, ref)
    got = host.sdpa(q, k, v, dt, **kw)
    check(i, c, capi.IMPL_AUTO, got, ref)
    return impls


WORST = {}       # dtype -> (absolute error, what): the largest error seen, for the log
# f32 checks that were granted a bar above 1e-5 (logits of 16 and more), and the plain ones beside them
WIDENED = {"checks": 0, "cases": set(), "worst": (0.0, 0.0, ""), "plain_checks": 0, "plain_worst": 0.0}


def check(i, c, impl, got, ref):
    what = "case %d impl %d %s" % (i, impl, {k: (v if not isinstance(v, np.ndarray) else v.shape) for k, v in c.items()})
    nr = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nr), what + ": NaN pattern"
    err = float(np.abs(np.where(nr, 0, got) - np.where(nr, 0, ref)).max()) if got.size else 0.0
    big = float(np.abs(np.where(nr, 0, ref)).max()) if got.size else 0.0
    if err > WORST.get(c["dtype"], (-1.0, ""))[0]:
        WORST[c["dtype"]] = (err, "%s (outputs up to %.2f)" % (what, big))
    if c["dtype"] == capi.F32:
        # absolute 1e-5 - except where the f32 representation of the logits themselves is coarser than that: the
        # reference narrows each f64-accumulated dot product to f32 (cpu/ops/matmul.rs:516-527), an error of 2^-24 |x| per
        # logit that reaches the output multiplied by the output's magnitude, so two faithful f32 evaluations differ by a
        # few times 2^-24 max|x| max|o| (drawn scales put |x| near 40 with |o| near 4: 4e-5).  N(0,1) operands at the
        # default scale stay far below the absolute bar.
        # The widened bar is only ever granted to cases whose logits reach 16 (N(0,1) operands at the default scale stay
        # below 8); every other f32 case is held to the plain 1e-5, and the log says how many cases were widened and what
        # their worst error was.
        bar = TOL[capi.F32]
        if c["max_logit"] >= 16.0:
            bar = max(bar, 4.0 * 2.0 ** -24 * c["max_logit"] * big)
        if bar > TOL[capi.F32]:
            WIDENED["checks"] += 1
            WIDENED["cases"].add(i)
            if err > WIDENED["worst"][0]:
                WIDENED["worst"] = (err, bar, what)
        else:
            WIDENED["plain_checks"] += 1
            WIDENED["plain_worst"] = max(WIDENED["plain_worst"], err)
    else:
        # 16-bit outputs: the stated bar (2e-2) is absolute and meant for outputs of order one, as the default scale gives;
        # a drawn scale several times the default makes the softmax pick single values of v (|o| up to ~4), where one
        # bf16 rounding of the output is already 8e-3: there the bar scales with the largest output magnitude.
        bar = TOL[c["dtype"]] * max(1.0, big)
    assert err <= bar, "%s: %.3e (outputs up to %.2f)" % (what, err, big)


def test_random_cases(gpu):
    r = np.random.Generator(np.random.PCG64(20261125))
    used = {}
    for i in range(N_CASES):
        c = draw_case(r)
        if i % 20 == 0:
            say("random case %d/%d" % (i, N_CASES))
        for impl in run_case(i, c, r):
            used[impl] = used.get(impl, 0) + 1
    say("kernels exercised: %s" % used)
    for dt, (err, what) in sorted(WORST.items()):
        say("worst absolute error, dtype %d: %.3e in %s" % (dt, err, what))
    say("f32: %d checks at the plain 1e-5 bar (worst %.3e); %d checks of %d cases with logits >= 16 at a widened bar "
        "(worst %.3e against its bar %.3e: %s)" % (WIDENED["plain_checks"], WIDENED["plain_worst"], WIDENED["checks"],
                                                   len(WIDENED["cases"]), WIDENED["worst"][0], WIDENED["worst"][1], WIDENED["worst"][2]))
    assert WIDENED["plain_checks"] > 4 * WIDENED["checks"], "the widened bar is the exception, not the rule"
    for impl in (capi.IMPL_GENERIC, capi.IMPL_MFMA, capi.IMPL_SPLITKV, capi.IMPL_SPLITKV_MFMA):
        assert used.get(impl, 0) >= 5, "kernel %d was hardly reached: %s" % (impl, used)


def test_random_cases_over_head_dimensions(gpu):
    """The same draw over the head dimensions the matrix-core kernels take padded (whole 16-byte vectors up to 128, above
    128 up to 256, D != Dv) and some they do not (rows of 4 or 12 bytes more than a vector), every kernel the planner
    accepts for each case."""
    r = np.random.Generator(np.random.PCG64(20261126))
    used = {}
    for i in range(80):
        c = draw_case(r, head_dims=(8, 24, 40, 72, 96, 104, 120, 136, 160, 192, 200, 248, 20, 132), other_dv=(8, 48, 96, 144, 256))
        if i % 20 == 0:
            say("random case (head dimensions) %d/80" % i)
        for impl in run_case(1000 + i, c, r):
            used[impl] = used.get(impl, 0) + 1
    say("kernels exercised: %s" % used)
    for impl in (capi.IMPL_GENERIC, capi.IMPL_MFMA, capi.IMPL_SPLITKV_MFMA):
        assert used.get(impl, 0) >= 5, "kernel %d was hardly reached: %s" % (impl, used)


def test_random_cases_with_masks_whose_rows_can_be_copied(gpu):
    """The same differential draw aimed at the path that takes a 16-bit mask's values through LDS (key counts that are
    multiples of 8, so that the mask's rows are 16-byte aligned): every case has a mask - values with holes, or blocks of 32 x 32
    that are hidden, zero or valued at random, or a band - with any of its leading axes broadcast, under the causal flag and key
    counts or not, query counts that do not fill the workgroups, grouped queries, head dimensions the instances take whole and
    padded; every kernel the planner accepts for each case."""
    r = np.random.Generator(np.random.PCG64(20261127))
    used = {}
    for i in range(60):
        dtype = int(r.choice([capi.F16, capi.BF16]))
        D = int(r.choice([64, 128, 128, 80, 32]))
        Dv = D if r.random() < 0.8 else int(r.choice([64, 128]))
        Hkv, G, B = int(r.integers(1, 4)), int(r.choice([1, 1, 2, 4])), int(r.integers(1, 4))
        Skv = 8 * int(r.integers(1, 90))
        Sq = Skv if r.random() < 0.5 else int(r.integers(1, 700))
        causal = bool(r.random() < 0.4)
        lens = r.integers(0, Skv + 1, B).astype(np.int32) if r.random() < 0.3 else None
        shp = [B if r.random() < 0.5 else 1, Hkv * G if r.random() < 0.5 else 1, Sq if r.random() < 0.8 else 1, Skv]
        kind = r.choice(["holes", "blocks", "band", "values"])
        mask = r.standard_normal(shp, dtype=np.float32)
        if kind == "holes":
            mask[r.random(shp) < 0.2] = -np.inf
        elif kind == "blocks":
            kinds = r.integers(0, 3, size=(shp[0], shp[1], (shp[2] + 31) // 32, (Skv + 31) // 32))
            big = np.repeat(np.repeat(kinds, 32, axis=2), 32, axis=3)[:, :, :shp[2], :Skv]
            mask = np.where(big == 0, -np.inf, np.where(big == 1, 0.0, mask)).astype(np.float32)
        elif kind == "band" and shp[2] > 1:
            dist = np.arange(Sq)[:, None] + (Skv - Sq) - np.arange(Skv)[None, :]
            mask = np.where((np.abs(dist) <= int(r.integers(8, 200)))[None, None], 0.1 * mask, -np.inf).astype(np.float32)
        c = dict(dtype=dtype, B=B, Hkv=Hkv, G=G, Sq=Sq, Skv=Skv, D=D, Dv=Dv, causal=causal, lens=lens, mask=mask,
                 scale=None if r.random() < 0.6 else float(r.uniform(0.02, 0.4)))
        if i % 20 == 0:
            say("random case (copyable masks) %d/60" % i)
        for impl in run_case(2000 + i, c, r):
            used[impl] = used.get(impl, 0) + 1
    say("kernels exercised: %s" % used)
    assert used.get(capi.IMPL_MFMA, 0) >= 40, "the prefill kernels were hardly reached: %s" % used
