"""incin_rocm_sdpa_fwd_static, the launch that takes its scratch memory from the library's static device buffer instead
of a workspace of the caller's: its output must equal incin_rocm_sdpa_fwd's bit for bit, on two calls in a row of which
the second is the smaller one (the buffer keeps the first call's contents), for the three launches that use scratch
memory: split-KV decode (partial results), a prefill launch over key splits (the same) and a matrix-core prefill with a
dense mask (block flags of the mask)."""
import sys

import numpy as np
import pytest

from incin_amd import capi, dtypes, host

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, file=sys.stderr, flush=True)


class Problem:
    def __init__(self, seed, B, Hq, Hkv, Sq, Skv, D, causal, impl, num_splits=0, kv_lens=None, causal_mask_tensor=False):
        r = np.random.Generator(np.random.PCG64(seed))
        mk = lambda *s: dtypes.round_to(r.standard_normal(s, dtype=np.float32), capi.BF16)
        self.tq, self.tk, self.tv = (host.DeviceTensor.from_f32(x, capi.BF16) for x in
                                     (mk(B, Hq, Sq, D), mk(B, Hkv, Skv, D), mk(B, Hkv, Skv, D)))
        self.to = host.DeviceTensor((B, Hq, Sq, D), capi.BF16)
        self.lens = capi.DeviceBuffer.from_numpy(np.asarray(kv_lens, dtype=np.int32)) if kv_lens is not None else None
        self.tm, ms = None, None
        if causal_mask_tensor:
            m = np.triu(np.full((Sq, Skv), -np.inf, np.float32), 1 + Skv - Sq)
            self.tm, ms = capi.DeviceBuffer.from_numpy(dtypes.encode(m, capi.BF16)), (0, 0, Skv, 1)
        self.desc = host.make_desc(self.tq, self.tk, self.tv, self.to, causal=causal, impl=impl, num_splits=num_splits,
                                   kv_lens=self.lens, mask=self.tm, mask_strides=ms)
        self.nbytes, self.splits, self.impl = capi.sdpa_workspace(self.desc)
        assert self.impl == impl and self.nbytes > 0

    def clear(self):
        capi.check(capi.load().incin_rocm_memset(0, self.to.ptr, 0xFF, self.to.buf.nbytes))
        capi.sync()

    def with_workspace(self):
        ws = capi.DeviceBuffer(self.nbytes)
        capi.check(capi.load().incin_rocm_memset(0, ws.ptr, 0xA5, ws.nbytes))     # a workspace needs no initialisation
        self.desc.workspace, self.desc.workspace_bytes = ws.ptr, ws.nbytes
        self.clear()
        capi.sdpa_fwd(self.desc)
        capi.sync()
        out = self.to.to_f32()
        self.desc.workspace, self.desc.workspace_bytes = None, 0
        ws.free()
        return out

    def static(self):
        self.clear()
        capi.sdpa_fwd_static(self.desc)
        capi.sync()
        return self.to.to_f32()


def test_static_scratch_matches_workspace_launch(gpu):
    big_small = [
        ("split-KV decode",
         dict(B=4, Hq=8, Hkv=8, Sq=1, Skv=4096, D=128, causal=False, impl=capi.IMPL_SPLITKV, num_splits=8),
         dict(B=2, Hq=4, Hkv=2, Sq=1, Skv=1500, D=128, causal=False, impl=capi.IMPL_SPLITKV, num_splits=3, kv_lens=[1500, 700])),
        ("matrix-core split-KV decode",
         dict(B=2, Hq=16, Hkv=2, Sq=1, Skv=4096, D=128, causal=False, impl=capi.IMPL_SPLITKV_MFMA, num_splits=8),
         dict(B=2, Hq=12, Hkv=2, Sq=3, Skv=1500, D=128, causal=True, impl=capi.IMPL_SPLITKV_MFMA, num_splits=3, kv_lens=[1500, 700])),
        ("prefill with the keys split",
         dict(B=1, Hq=4, Hkv=2, Sq=100, Skv=4500, D=128, causal=True, impl=capi.IMPL_MFMA),
         dict(B=1, Hq=2, Hkv=2, Sq=40, Skv=4100, D=128, causal=False, impl=capi.IMPL_MFMA, num_splits=3)),
        ("prefill with a dense mask (block flags)",
         dict(B=2, Hq=4, Hkv=2, Sq=700, Skv=700, D=128, causal=False, impl=capi.IMPL_MFMA, causal_mask_tensor=True),
         dict(B=1, Hq=2, Hkv=2, Sq=100, Skv=333, D=128, causal=False, impl=capi.IMPL_MFMA, causal_mask_tensor=True)),
        ("matrix-core split-KV decode, head dimensions padded to the 256 and the 128 instance (partial rows that wide)",
         dict(B=2, Hq=16, Hkv=2, Sq=1, Skv=4096, D=192, causal=False, impl=capi.IMPL_SPLITKV_MFMA, num_splits=8),
         dict(B=2, Hq=12, Hkv=2, Sq=3, Skv=1500, D=96, causal=True, impl=capi.IMPL_SPLITKV_MFMA, num_splits=3, kv_lens=[1500, 700])),
        ("prefill with the keys split, head dimension 112 (128 instance) then 40 (64 instance)",
         dict(B=1, Hq=4, Hkv=2, Sq=100, Skv=4500, D=112, causal=True, impl=capi.IMPL_MFMA),
         dict(B=1, Hq=2, Hkv=2, Sq=40, Skv=4100, D=40, causal=False, impl=capi.IMPL_MFMA, num_splits=3)),
    ]
    for name, big, small in big_small:
        pb, ps = Problem(7, **big), Problem(8, **small)
        want_big, want_small = pb.with_workspace(), ps.with_workspace()
        assert np.isfinite(want_big).all() and np.isfinite(want_small).all()
        say("%s: static scratch, large then small" % name)
        got_big = pb.static()
        got_small = ps.static()
        assert np.array_equal(got_big, want_big), name
        assert np.array_equal(got_small, want_small), name
        got_big = pb.static()                            # and the large one again over the small one's leftovers
        assert np.array_equal(got_big, want_big), name


def test_static_scratch_limit_and_no_workspace_needed(gpu):
    # a request beyond the buffer is refused, with the workspace launch named as the way out
    p = Problem(9, B=64, Hq=32, Hkv=32, Sq=1, Skv=8192, D=128, causal=False, impl=capi.IMPL_SPLITKV, num_splits=16)
    assert p.nbytes > capi.STATIC_SCRATCH_BYTES
    with pytest.raises(capi.RocmError) as e:
        capi.sdpa_fwd_static(p.desc)
    assert e.value.code == capi.EWORKSPACE and "static buffer" in str(e.value)
    # kernels without scratch memory run through the same entry point
    r = np.random.Generator(np.random.PCG64(3))
    mk = lambda *s: dtypes.round_to(r.standard_normal(s, dtype=np.float32), capi.BF16)
    q, k, v = mk(1, 2, 200, 128), mk(1, 2, 200, 128), mk(1, 2, 200, 128)
    want = host.sdpa(q, k, v, capi.BF16, causal=True)
    tq, tk, tv = (host.DeviceTensor.from_f32(x, capi.BF16) for x in (q, k, v))
    to = host.DeviceTensor((1, 2, 200, 128), capi.BF16)
    d = host.make_desc(tq, tk, tv, to, causal=True)
    capi.sdpa_fwd_static(d)
    capi.sync()
    assert np.array_equal(to.to_f32(), want)


def test_static_scratch_takes_a_prefill_launch_whole_when_its_partials_do_not_fit(gpu):
    """The library would split the keys of this launch (few row blocks, many keys) and the splits' partial results
    exceed the static buffer: the entry point runs the launch unsplit - no scratch memory needed - instead of refusing."""
    B, Hq, Hkv, Sq, Skv, D = 1, 32, 8, 256, 16384, 128
    r = np.random.Generator(np.random.PCG64(5))
    mk = lambda *s: dtypes.round_to(r.standard_normal(s, dtype=np.float32), capi.BF16)
    q, k, v = mk(B, Hq, Sq, D), mk(B, Hkv, Skv, D), mk(B, Hkv, Skv, D)
    tq, tk, tv = (host.DeviceTensor.from_f32(x, capi.BF16) for x in (q, k, v))
    to = host.DeviceTensor((B, Hq, Sq, D), capi.BF16)
    d = host.make_desc(tq, tk, tv, to, causal=True)
    nbytes, splits, impl = capi.sdpa_workspace(d)
    assert impl == capi.IMPL_MFMA and splits > 1 and nbytes > capi.STATIC_SCRATCH_BYTES
    capi.sdpa_fwd_static(d)
    capi.sync()
    got = to.to_f32()
    whole = host.sdpa(q, k, v, capi.BF16, causal=True, impl=capi.IMPL_MFMA, num_splits=1)
    assert np.array_equal(got, whole)
    # a forced split count beyond the buffer is refused as before
    d.num_splits = splits
    with pytest.raises(capi.RocmError) as e:
        capi.sdpa_fwd_static(d)
    assert e.value.code == capi.EWORKSPACE
