"""Decode loop over a key/value cache kept on the device: per token, incin_rocm_kv_append writes the token's K and V
rows at kv_lens[b] and advances the counts, incin_rocm_sdpa_fwd attends over the cache with the same kv_lens.  The
step is recorded into a launch graph once and replayed per token; nothing comes from the host in between.  Token t
of sequence b must equal row start[b] + t of causal attention over the whole sequence (the oracle)."""
import sys

import numpy as np
import pytest

from incin_amd import capi, dtypes, host
from oracle import oracle as O

pytestmark = pytest.mark.gpu
TOL = {capi.F32: 1e-5, capi.BF16: 2e-2}


def say(msg):
    print(msg, file=sys.stderr, flush=True)


def strides3(shape):
    B, H, S, D = shape
    return (H * S * D, S * D, D)


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F32])
@pytest.mark.parametrize("replay", [False, True], ids=["eager", "graph"])
def test_decode_loop_over_a_device_side_cache(gpu, dtype, replay):
    B, Hq, Hkv, D, S_max, T = 3, 8, 2, 128, 320, 24
    start = np.array([200, 0, 295], np.int32)             # tokens already in the cache; 295 + 24 runs to S_max - 1
    r = np.random.Generator(np.random.PCG64(77))
    mk = lambda *s: dtypes.round_to(r.standard_normal(s, dtype=np.float32), dtype)
    q_all, k_all, v_all = mk(B, Hq, S_max, D), mk(B, Hkv, S_max, D), mk(B, Hkv, S_max, D)
    say("decode loop: dtype %d, %s, starts %s, %d tokens" % (dtype, "graph replay" if replay else "eager", start.tolist(), T))

    # caches hold the prefix of each sequence; what lies beyond kv_lens is garbage the kernels must not read as data
    k_cache, v_cache = mk(B, Hkv, S_max, D) * 50, mk(B, Hkv, S_max, D) * 50
    for b in range(B):
        k_cache[b, :, :start[b]] = k_all[b, :, :start[b]]
        v_cache[b, :, :start[b]] = v_all[b, :, :start[b]]
    tkc, tvc = host.DeviceTensor.from_f32(k_cache, dtype), host.DeviceTensor.from_f32(v_cache, dtype)
    lens = capi.DeviceBuffer.from_numpy(start.copy())
    # per-token inputs live in fixed device buffers the host refills between steps (a model would write them)
    tq, tkn, tvn = (host.DeviceTensor((B, H, 1, D), dtype) for H in (Hq, Hkv, Hkv))
    to = host.DeviceTensor((B, Hq, 1, D), dtype)

    ad = capi.KvAppendDesc()
    ad.dtype, ad.device = dtype, 0
    ad.B, ad.Hkv, ad.S_new, ad.S_max, ad.D, ad.Dv = B, Hkv, 1, S_max, D, D
    ad.k_new, ad.v_new, ad.k_cache, ad.v_cache, ad.kv_lens = tkn.ptr, tvn.ptr, tkc.ptr, tvc.ptr, lens.ptr
    for name, shape in (("k_new_stride", (B, Hkv, 1, D)), ("v_new_stride", (B, Hkv, 1, D)),
                        ("k_cache_stride", (B, Hkv, S_max, D)), ("v_cache_stride", (B, Hkv, S_max, D))):
        for i, s in enumerate(strides3(shape)):
            getattr(ad, name)[i] = s
    sd = host.make_desc(tq, tkc, tvc, to, kv_lens=lens)
    nbytes, _, impl = capi.sdpa_workspace(sd)
    ws = capi.DeviceBuffer(nbytes) if nbytes else None
    if ws is not None:
        sd.workspace, sd.workspace_bytes = ws.ptr, ws.nbytes
    # 4 query heads per KV head: the matrix-core split-KV kernels (16-bit and f32)
    assert impl == capi.IMPL_SPLITKV_MFMA

    stream = capi.Stream()
    graph = None
    if replay:
        with capi.Graph.record(stream) as graph:
            capi.kv_append(ad, stream.ptr)
            capi.sdpa_fwd(sd, stream.ptr)

    enc = lambda x: dtypes.encode(np.ascontiguousarray(x), dtype)
    outs = np.zeros((B, Hq, T, D), np.float32)
    for t in range(T):
        pos = start + t
        for dst, src in ((tq, q_all), (tkn, k_all), (tvn, v_all)):
            raw = enc(np.stack([src[b, :, pos[b]:pos[b] + 1] for b in range(B)]))      # kept alive across the copy
            capi.check(capi.load().incin_rocm_memcpy_h2d(0, dst.ptr, raw.ctypes.data, raw.nbytes))
        if replay:
            graph.launch()
        else:
            capi.kv_append(ad, stream.ptr)
            capi.sdpa_fwd(sd, stream.ptr)
        stream.sync()
        outs[:, :, t] = to.to_f32()[:, :, 0]
    assert lens.to_numpy(np.int32, (B,)).tolist() == np.minimum(start + T, S_max).tolist()

    # oracle: causal attention over each whole sequence, rows start[b] .. start[b] + T - 1
    G = Hq // Hkv
    ref = O.sdpa(q_all.reshape(B, Hkv, G, S_max, D), k_all[:, :, None], v_all[:, :, None], causal=True).reshape(B, Hq, S_max, D)
    for b in range(B):
        want = ref[b, :, start[b]:start[b] + T]
        err = float(np.abs(outs[b] - want).max())
        say("   sequence %d: max-abs err %.3e" % (b, err))
        assert err <= TOL[dtype]
    # the cache now holds the sequences' rows, bit for bit
    kc = tkc.to_f32()
    for b in range(B):
        n = min(start[b] + T, S_max)
        assert np.array_equal(kc[b, :, :n], k_all[b, :, :n])
    if graph is not None:
        graph.destroy()


def test_append_many_rows_strided_and_full_cache(gpu):
    # several rows at once, D != Dv, f32 rows that are not multiples of 16 bytes, a cache that fills up
    B, Hkv, S_new, S_max, D, Dv = 2, 3, 5, 12, 6, 10
    r = np.random.Generator(np.random.PCG64(78))
    kn, vn = r.standard_normal((B, Hkv, S_new, D), dtype=np.float32), r.standard_normal((B, Hkv, S_new, Dv), dtype=np.float32)
    kc, vc = np.zeros((B, Hkv, S_max, D), np.float32), np.zeros((B, Hkv, S_max, Dv), np.float32)
    start = np.array([2, 9], np.int32)                     # the second sequence has room for 3 of the 5 rows
    tkn, tvn, tkc, tvc = (host.DeviceTensor.from_f32(x, capi.F32) for x in (kn, vn, kc, vc))
    lens = capi.DeviceBuffer.from_numpy(start.copy())
    ad = capi.KvAppendDesc()
    ad.dtype, ad.device = capi.F32, 0
    ad.B, ad.Hkv, ad.S_new, ad.S_max, ad.D, ad.Dv = B, Hkv, S_new, S_max, D, Dv
    ad.k_new, ad.v_new, ad.k_cache, ad.v_cache, ad.kv_lens = tkn.ptr, tvn.ptr, tkc.ptr, tvc.ptr, lens.ptr
    for name, shape in (("k_new_stride", kn.shape), ("v_new_stride", vn.shape), ("k_cache_stride", kc.shape), ("v_cache_stride", vc.shape)):
        for i, s in enumerate(strides3(shape)):
            getattr(ad, name)[i] = s
    capi.kv_append(ad)
    capi.sync()
    gk, gv = tkc.to_f32(), tvc.to_f32()
    for b in range(B):
        n = min(S_new, S_max - start[b])
        assert np.array_equal(gk[b, :, start[b]:start[b] + n], kn[b, :, :n])
        assert np.array_equal(gv[b, :, start[b]:start[b] + n], vn[b, :, :n])
        assert not gk[b, :, :start[b]].any() and not gk[b, :, start[b] + n:].any()
    assert lens.to_numpy(np.int32, (B,)).tolist() == [7, 12]
    # errors are reported, not executed
    ad.dtype = 9
    with pytest.raises(capi.RocmError) as e:
        capi.kv_append(ad)
    assert e.value.code == capi.EDTYPE
