"""The launch path under conditions a serving loop puts it in: several host threads launching on streams of their
own at once (the C ABI promises this is safe), and launches captured into a HIP graph and replayed (the launch path
neither allocates nor clears memory).  Results must equal the plain launch bit for bit."""
import sys
import threading

import numpy as np
import pytest

from incin_amd import capi, dtypes, host

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, file=sys.stderr, flush=True)


class Case:
    def __init__(self, seed, B, Hq, Hkv, Sq, Skv, D, causal, impl, dtype=capi.BF16, banded_mask=False):
        r = np.random.Generator(np.random.PCG64(seed))
        mk = lambda *s: dtypes.round_to(r.standard_normal(s, dtype=np.float32), dtype)
        self.tq, self.tk, self.tv = (host.DeviceTensor.from_f32(x, dtype) for x in
                                     (mk(B, Hq, Sq, D), mk(B, Hkv, Skv, D), mk(B, Hkv, Skv, D)))
        self.to = host.DeviceTensor((B, Hq, Sq, D), dtype)
        self.tm, ms = None, None
        if banded_mask:         # a [Sq, Skv] additive tensor: values near the diagonal, -inf away from it, zeros between
            d = np.abs(np.arange(Sq)[:, None] - np.arange(Skv)[None, :])
            m = np.where(d > 200, -np.inf, np.where(d < 40, r.standard_normal((Sq, Skv)), 0.0)).astype(np.float32)
            self.tm, ms = capi.DeviceBuffer.from_numpy(dtypes.encode(dtypes.round_to(m, dtype), dtype)), (0, 0, Skv, 1)
        self.desc = host.make_desc(self.tq, self.tk, self.tv, self.to, causal=causal, impl=impl, mask=self.tm, mask_strides=ms)
        nbytes, _, self.impl = capi.sdpa_workspace(self.desc)
        self.ws = capi.DeviceBuffer(nbytes) if nbytes else None
        if self.ws is not None:
            self.desc.workspace, self.desc.workspace_bytes = self.ws.ptr, self.ws.nbytes

    def plain(self):
        capi.sdpa_fwd(self.desc)
        capi.sync()
        return self.to.to_f32()

    def clear(self):
        capi.check(capi.load().incin_rocm_memset(0, self.to.ptr, 0xFF, self.to.buf.nbytes))
        capi.sync()


CASES = [
    ("prefill 32-row kernel", dict(B=2, Hq=8, Hkv=8, Sq=512, Skv=512, D=128, causal=True, impl=capi.IMPL_MFMA)),
    ("prefill over key splits", dict(B=1, Hq=4, Hkv=2, Sq=128, Skv=4200, D=128, causal=True, impl=capi.IMPL_MFMA)),
    ("decode split-KV", dict(B=4, Hq=8, Hkv=8, Sq=1, Skv=4096, D=128, causal=False, impl=capi.IMPL_SPLITKV)),
    ("grouped-query decode, matrix-core split-KV", dict(B=2, Hq=16, Hkv=2, Sq=1, Skv=4096, D=128, causal=False, impl=capi.IMPL_SPLITKV_MFMA)),
    ("generic", dict(B=1, Hq=2, Hkv=2, Sq=100, Skv=130, D=80, causal=True, impl=capi.IMPL_GENERIC)),
    ("f32 matrix-core prefill", dict(B=2, Hq=4, Hkv=2, Sq=300, Skv=300, D=64, causal=True, impl=capi.IMPL_MFMA, dtype=capi.F32)),
    ("prefill with a dense mask", dict(B=1, Hq=4, Hkv=4, Sq=512, Skv=512, D=128, causal=False, impl=capi.IMPL_MFMA, banded_mask=True)),
]


def test_threads_on_their_own_streams(gpu):
    cases = [Case(100 + i, **kw) for i, (_, kw) in enumerate(CASES)]
    expect = [c.plain() for c in cases]
    for c in cases:
        c.clear()
    errors = []

    def worker(c):
        try:
            s = capi.Stream()
            for _ in range(25):
                capi.sdpa_fwd(c.desc, s.ptr)
            s.sync()
        except Exception as e:      # noqa: BLE001 - reported below
            errors.append(e)

    say("%d threads x 25 launches, one stream and one kernel each" % len(cases))
    threads = [threading.Thread(target=worker, args=(c,)) for c in cases]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for (name, _), c, e in zip(CASES, cases, expect):
        got = c.to.to_f32()
        assert np.array_equal(np.nan_to_num(got, nan=3.0), np.nan_to_num(e, nan=3.0)), name


@pytest.mark.parametrize("name, kw", CASES, ids=[n for n, _ in CASES])
def test_graph_capture_and_replay(gpu, name, kw):
    c = Case(200, **kw)
    expect = c.plain()
    say("graph capture: %s" % name)
    stream = capi.Stream()
    with capi.Graph.record(stream) as graph:
        capi.sdpa_fwd(c.desc, stream.ptr)
        capi.sdpa_fwd(c.desc, stream.ptr)          # twice in one graph: the second must see what the first leaves behind
    for replay in range(3):
        c.clear()
        graph.launch()
        stream.sync()
        got = c.to.to_f32()
        assert np.array_equal(np.nan_to_num(got, nan=3.0), np.nan_to_num(expect, nan=3.0)), "%s, replay %d" % (name, replay)
        # eager work of the program's own between replays
        assert np.array_equal(np.nan_to_num(c.plain(), nan=3.0), np.nan_to_num(expect, nan=3.0))
    graph.destroy()


@pytest.mark.parametrize("dtype, impl, S, heads", [(capi.BF16, capi.IMPL_AUTO, 300, (4, 2)), (capi.F32, capi.IMPL_AUTO, 300, (4, 2)),
                                                   (capi.F32, capi.IMPL_AUTO, 1100, (4, 2)), (capi.F32, capi.IMPL_GENERIC, 300, (4, 2)),
                                                   (capi.BF16, capi.IMPL_AUTO, 1100, (8, 1))],
                         ids=["bf16_matrix_core", "f32_matrix_core", "f32_matrix_core_dealt_blocks", "f32_generic", "bf16_one_kv_head_dealt_walks"])
def test_training_step_in_a_graph(gpu, dtype, impl, S, heads):
    """Forward (keeping the row normalisers) and backward recorded into one launch graph and replayed: every replay gives
    the bytes the eager calls gave, with the program's own eager work between replays.  The backward launches three kernels
    (up to five at 1100 tokens, where the walks of a block - in f32, and in bf16 with eight query heads on one KV head - are dealt to
    several workgroups and a pass adds their sums) on
    the captured stream alone - eagerly a call this small puts one of them on a second stream - and neither allocates nor
    clears memory."""
    (Hq, Hkv), B, D = heads, 2, 128
    r = np.random.Generator(np.random.PCG64(300))
    mk = lambda *s: r.standard_normal(s, dtype=np.float32)
    tq, tk, tv, tg = (host.DeviceTensor.from_f32(x, dtype) for x in (mk(B, Hq, S, D), mk(B, Hkv, S, D), mk(B, Hkv, S, D), mk(B, Hq, S, D)))
    to, tdq = host.DeviceTensor((B, Hq, S, D), dtype), host.DeviceTensor((B, Hq, S, D), dtype)
    tdk, tdv = host.DeviceTensor((B, Hkv, S, D), dtype), host.DeviceTensor((B, Hkv, S, D), dtype)
    lse = capi.DeviceBuffer(B * Hq * S * 4)
    bd = capi.SdpaBwdDesc()
    bd.fwd = host.make_desc(tq, tk, tv, to, causal=True, impl=impl, lse=lse)
    fws = capi.DeviceBuffer(max(capi.sdpa_workspace(bd.fwd)[0], 256))
    bd.fwd.workspace, bd.fwd.workspace_bytes = fws.ptr, fws.nbytes
    for name, t in (("d_o", tg), ("d_q", tdq), ("d_k", tdk), ("d_v", tdv)):
        setattr(bd, name, t.ptr)
        st = host._strides3(t.shape)
        for i in range(3):
            getattr(bd, name + "_stride")[i] = st[i]
    ws = capi.DeviceBuffer(capi.sdpa_bwd_workspace(bd))
    bd.workspace, bd.workspace_bytes = ws.ptr, ws.nbytes
    outs = (to, tdq, tdk, tdv)

    def eager():
        capi.sdpa_fwd(bd.fwd)
        capi.sdpa_bwd(bd)
        capi.sync()
        return [t.to_f32() for t in outs]

    def clear():
        for t in outs:
            capi.check(capi.load().incin_rocm_memset(0, t.ptr, 0x7f, t.buf.nbytes))
        capi.sync()

    expect = eager()
    say("graph capture: forward + backward, dtype %d" % dtype)
    stream = capi.Stream()
    with capi.Graph.record(stream) as graph:
        capi.sdpa_fwd(bd.fwd, stream.ptr)
        capi.sdpa_bwd(bd, stream.ptr)
    for replay in range(3):
        clear()
        graph.launch()
        stream.sync()
        for name, t, e in zip(("out", "dq", "dk", "dv"), outs, expect):
            assert np.array_equal(t.to_f32(), e), "%s, replay %d" % (name, replay)
        for got, e in zip(eager(), expect):          # eager work of the program's own between replays
            assert np.array_equal(got, e)
    graph.destroy()
    stream.destroy()


def test_overlapping_launches_with_workspaces_of_their_own(gpu):
    """Two host threads launch the same problem - grouped-query decode through the matrix-core split-KV kernel, whose
    splits leave their partial results in the launch's workspace for the combine pass - 50 times each on streams of their
    own while a recorded graph of the same launch replays on a third stream.  Each party has a workspace and an output
    of its own, so whatever overlaps, every output equals the plain launch bit for bit."""
    kw = dict(B=2, Hq=16, Hkv=2, Sq=1, Skv=6000, D=128, causal=False, impl=capi.IMPL_SPLITKV_MFMA)
    parties = [Case(400, **kw) for _ in range(3)]          # same seed: same problem, separate buffers
    assert all(c.impl == capi.IMPL_SPLITKV_MFMA and c.ws is not None for c in parties)
    expect = parties[0].plain()
    for c in parties:
        c.clear()
    gstream = capi.Stream()
    with capi.Graph.record(gstream) as graph:
        capi.sdpa_fwd(parties[2].desc, gstream.ptr)
    errors = []

    def eager(c):
        try:
            s = capi.Stream()
            for _ in range(50):
                capi.sdpa_fwd(c.desc, s.ptr)
            s.sync()
            s.destroy()
        except Exception as e:      # noqa: BLE001 - reported below
            errors.append(e)

    def replay():
        try:
            for _ in range(50):
                graph.launch()
            gstream.sync()
        except Exception as e:      # noqa: BLE001
            errors.append(e)

    say("2 threads x 50 eager launches + 50 graph replays of a split-KV launch, three streams")
    threads = [threading.Thread(target=eager, args=(parties[0],)), threading.Thread(target=eager, args=(parties[1],)),
               threading.Thread(target=replay)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    capi.sync()
    for i, c in enumerate(parties):
        assert np.array_equal(c.to.to_f32(), expect), "party %d" % i
    graph.destroy()
    gstream.destroy()


class BackwardPair:
    """Two dependent backward calls: the second takes the first's dQ as its dO, so it is right only if the first call's
    kernels - whichever stream the library put them on - are ordered before it on the caller's stream."""

    def __init__(self, seed, dtype, D, B=2, Hq=4, Hkv=2, S=300):
        r = np.random.Generator(np.random.PCG64(seed))
        mk = lambda *s: r.standard_normal(s, dtype=np.float32)
        self.keep = []
        tq, tk, tv, tg = (host.DeviceTensor.from_f32(x, dtype) for x in (mk(B, Hq, S, D), mk(B, Hkv, S, D), mk(B, Hkv, S, D), mk(B, Hq, S, D)))
        to = host.DeviceTensor((B, Hq, S, D), dtype)
        lse = capi.DeviceBuffer(B * Hq * S * 4)
        fwd = host.make_desc(tq, tk, tv, to, causal=True, lse=lse)
        nbytes, _, _ = capi.sdpa_workspace(fwd)
        fws = capi.DeviceBuffer(max(nbytes, 256))
        fwd.workspace, fwd.workspace_bytes = fws.ptr, fws.nbytes
        capi.sdpa_fwd(fwd)
        capi.sync()
        self.keep += [tq, tk, tv, tg, to, lse, fws]
        self.outs, self.descs = [], []
        d_o = tg
        for _ in range(2):
            tdq = host.DeviceTensor((B, Hq, S, D), dtype)
            tdk, tdv = host.DeviceTensor((B, Hkv, S, D), dtype), host.DeviceTensor((B, Hkv, S, D), dtype)
            bd = capi.SdpaBwdDesc()
            bd.fwd = fwd
            for name, t in (("d_o", d_o), ("d_q", tdq), ("d_k", tdk), ("d_v", tdv)):
                setattr(bd, name, t.ptr)
                st = host._strides3(t.shape)
                for i in range(3):
                    getattr(bd, name + "_stride")[i] = st[i]
            ws = capi.DeviceBuffer(capi.sdpa_bwd_workspace(bd))
            bd.workspace, bd.workspace_bytes = ws.ptr, ws.nbytes
            self.keep.append(ws)
            self.descs.append(bd)
            self.outs += [tdq, tdk, tdv]
            d_o = tdq

    def run(self, stream=None):
        for bd in self.descs:
            capi.sdpa_bwd(bd, stream)

    def clear(self):
        for t in self.outs:
            capi.check(capi.load().incin_rocm_memset(0, t.ptr, 0x7f, t.buf.nbytes))
        capi.sync()

    def read(self):
        return [t.to_f32() for t in self.outs]


@pytest.mark.parametrize("dtype, D", [(capi.BF16, 128), (capi.BF16, 64), (capi.F32, 128), (capi.F32, 64)],
                         ids=["bf16_d128", "bf16_d64", "f32_d128", "f32_d64"])
def test_backward_with_its_dq_kernel_on_a_side_stream(gpu, dtype, D, monkeypatch):
    """A backward call short of work puts its dQ kernel on a stream of the library's own beside the dK/dV kernel and joins
    the caller's stream afterwards.  Against the same calls held to one stream (INCIN_ROCM_BWD_STREAMS=1): bit-identical
    gradients of two dependent calls, back to back on a stream of the caller's, and from three host threads at once, each on
    a stream of its own with problems of its own (the library's streams come out of a shared pool)."""
    pairs = [BackwardPair(500 + i, dtype, D) for i in range(3)]
    monkeypatch.setenv("INCIN_ROCM_BWD_STREAMS", "1")
    expect = []
    for p in pairs:
        p.run()
        capi.sync()
        expect.append(p.read())
        p.clear()
    monkeypatch.delenv("INCIN_ROCM_BWD_STREAMS")
    say("backward on two streams: dtype %d, D %d, one thread" % (dtype, D))
    stream = capi.Stream()
    for rep in range(5):
        pairs[0].run(stream.ptr)
        stream.sync()
        for name, got, e in zip(("dq1", "dk1", "dv1", "dq2", "dk2", "dv2"), pairs[0].read(), expect[0]):
            assert np.array_equal(got, e), "%s, repetition %d" % (name, rep)
        pairs[0].clear()
    stream.destroy()
    errors = []

    def worker(p):
        try:
            s = capi.Stream()
            for _ in range(15):
                p.run(s.ptr)
            s.sync()
            s.destroy()
        except Exception as e:      # noqa: BLE001 - reported below
            errors.append(e)

    say("backward on two streams: dtype %d, D %d, three threads" % (dtype, D))
    threads = [threading.Thread(target=worker, args=(p,)) for p in pairs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    capi.sync()
    for i, (p, exp) in enumerate(zip(pairs, expect)):
        for name, got, e in zip(("dq1", "dk1", "dv1", "dq2", "dk2", "dv2"), p.read(), exp):
            assert np.array_equal(got, e), "thread %d, %s" % (i, name)
