"""CPU-side checks of the C ABI: the library loads, exports every symbol the header
declares, the descriptor layout matches the ctypes mirror, and descriptor
validation (which runs before any device call) reports the documented codes."""
import ctypes as C
import os
import re

import pytest

from incin_amd import capi

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "incin_rocm.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(incin_rocm_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    names = declared_functions()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), "missing export %s" % n
    assert set(names) == set(capi.EXPORTS)
    assert lib.incin_rocm_abi_version() == 11


def test_descriptor_layout_matches():
    lib = capi.load()
    lib.incin_rocm_sizeof_sdpa_desc.restype = C.c_size_t
    assert lib.incin_rocm_sizeof_sdpa_desc() == C.sizeof(capi.SdpaDesc)
    lib.incin_rocm_sizeof_device_info.restype = C.c_size_t
    assert lib.incin_rocm_sizeof_device_info() == C.sizeof(capi.DeviceInfo)


def _desc(**kw):
    d = capi.SdpaDesc()
    d.dtype, d.device = capi.BF16, 0
    d.B, d.Hq, d.Hkv, d.Sq, d.Skv, d.D, d.Dv = 2, 4, 4, 128, 128, 128, 128
    for name in ("q_stride", "k_stride", "v_stride", "o_stride"):
        st = getattr(d, name)
        st[0], st[1], st[2] = 4 * 128 * 128, 128 * 128, 128
    d.q = d.k = d.v = d.o = 0x10000          # never dereferenced by validation
    d.scale = 0.088
    for k, v in kw.items():
        setattr(d, k, v)
    return d


def _plan(d):
    return capi.sdpa_workspace(d)


def test_dispatch_choices():
    assert _plan(_desc())[2] == capi.IMPL_MFMA
    # f32: the IEEE-f32 matrix-core prefill kernel where the launch gives it more than two 128-row workgroups per compute unit
    # (256 compute units here: no device to ask), the f32 split-KV kernel - 32 rows per workgroup, keys dealt to its wavefronts,
    # two workgroups per compute unit - up to that
    assert _plan(_desc(dtype=capi.F32, B=8, Hq=16, Sq=4096, Skv=4096))[2] == capi.IMPL_MFMA
    assert _plan(_desc(dtype=capi.F32, B=4, Hq=8, Sq=1024, Skv=1024))[2] == capi.IMPL_SPLITKV_MFMA      # 4 x 8 heads x 1024 x 1024: 256 workgroups
    assert _plan(_desc(dtype=capi.F32, B=4, Hq=8, Sq=2048, Skv=2048))[2] == capi.IMPL_SPLITKV_MFMA      # 512
    assert _plan(_desc(dtype=capi.F32, B=4, Hq=8, Sq=2049, Skv=2049))[2] == capi.IMPL_MFMA              # 544
    assert _plan(_desc(dtype=capi.F32))[2] == capi.IMPL_SPLITKV_MFMA
    assert _plan(_desc(dtype=capi.F32, impl=capi.IMPL_MFMA))[2] == capi.IMPL_MFMA
    assert _plan(_desc(dtype=capi.F32, add_mask=0x20000))[2] == capi.IMPL_MFMA  # which also takes a dense mask
    # head dimensions up to 128 in whole 16-byte vectors (D and Dv need not be equal) run padded in the matrix-core kernels
    assert _plan(_desc(dtype=capi.F32, D=80, Dv=80, B=8, Hq=16, Sq=4096, Skv=4096))[2] == capi.IMPL_MFMA
    assert _plan(_desc(D=80, Dv=80))[2] == capi.IMPL_MFMA
    assert _plan(_desc(D=128, Dv=64))[2] == capi.IMPL_MFMA
    assert _plan(_desc(D=8, Dv=40))[2] == capi.IMPL_MFMA
    assert _plan(_desc(D=84, Dv=84))[2] == capi.IMPL_GENERIC                    # 168-byte rows: not whole vectors
    assert _plan(_desc(dtype=capi.F32, D=84, Dv=84, B=8, Hq=16, Sq=4096, Skv=4096))[2] == capi.IMPL_MFMA       # in f32 they are
    # above 128: 16-bit prefill shapes on the prefill kernel for 256, decode shapes (up to 64 positions) and f32 on the 256
    # instance of the matrix-core split-KV kernels
    assert _plan(_desc(D=160, Dv=160, B=64))[2] == capi.IMPL_MFMA
    assert _plan(_desc(D=128, Dv=136, B=64))[2] == capi.IMPL_MFMA
    # (launches that give that prefill kernel workgroups for at most half the compute units go 32 rows per workgroup through
    # the split-KV kernel - 8 workgroups here, then 128 over 3000 keys - unless the keys are long enough to be split so that
    # every compute unit gets a workgroup: 128 workgroups x 4 splits of 4096 keys, and a 256-row chunk of a 16384-token prompt)
    assert _plan(_desc(D=160, Dv=160))[2] == capi.IMPL_SPLITKV_MFMA
    assert _plan(_desc(D=256, Dv=256, B=1, Hq=16, Hkv=16, Sq=1024, Skv=3000, causal=1))[2] == capi.IMPL_SPLITKV_MFMA
    nbytes, splits, impl = _plan(_desc(D=256, Dv=256, B=1, Hq=16, Hkv=16, Sq=1024, Skv=4096, causal=1))
    assert impl == capi.IMPL_MFMA and splits == 4 and nbytes == 16 * 1024 * 4 * 258 * 4
    nbytes, splits, impl = _plan(_desc(D=256, Dv=256, B=1, Hq=32, Hkv=8, Sq=256, Skv=16384, causal=1))
    assert impl == capi.IMPL_MFMA and splits == 8
    assert _plan(_desc(D=256, Dv=256, B=1, Hq=8, Hkv=8, Sq=128, Skv=8192, causal=1))[2] == capi.IMPL_SPLITKV_MFMA      # 8 workgroups x 8 splits: not enough
    assert _plan(_desc(D=256, Dv=256, B=1, Hq=17, Hkv=17, Sq=1024, Skv=4096, causal=1))[2] == capi.IMPL_MFMA
    # (72 workgroups, 288 chunks of 32 rows: a ragged second round for the split-KV kernel, measured 1.25 times behind)
    assert _plan(_desc(D=256, Dv=256, B=1, Hq=12, Hkv=12, Sq=768, Skv=3000, causal=1))[2] == capi.IMPL_MFMA
    assert _plan(_desc(D=256, Dv=256, B=1, Hq=8, Hkv=8, Sq=768, Skv=3000, causal=1))[2] == capi.IMPL_SPLITKV_MFMA      # 48 workgroups
    assert _plan(_desc(D=256, Dv=256, B=1, Hq=8, Hkv=8, Sq=768, Skv=1024, causal=1))[2] == capi.IMPL_MFMA              # over 1024 keys: 192 chunks, one ragged round
    assert _plan(_desc(D=256, Dv=256, Sq=4096, Skv=4096, causal=1))[2] == capi.IMPL_MFMA
    assert _plan(_desc(D=256, Dv=256, Sq=4096, Skv=4096, causal=1, impl=capi.IMPL_SPLITKV_MFMA))[2] == capi.IMPL_SPLITKV_MFMA
    assert _plan(_desc(D=256, Dv=256, Sq=64, Skv=4096, causal=1))[2] == capi.IMPL_SPLITKV_MFMA
    assert _plan(_desc(D=256, Dv=256, Sq=1, Skv=4096, Hkv=1))[2] == capi.IMPL_SPLITKV_MFMA
    assert _plan(_desc(dtype=capi.F32, D=160, Dv=160))[2] == capi.IMPL_SPLITKV_MFMA
    # decode over such a cache: the matrix-core split-KV kernels, also at one row per KV head (no vector-ALU kernel there);
    # partial rows are as wide as the kernel instance
    nbytes, splits, impl = _plan(_desc(Sq=1, Skv=8192, B=2, Hq=8, Hkv=8, D=96, Dv=96, num_splits=4))
    assert impl == capi.IMPL_SPLITKV_MFMA and splits == 4 and nbytes == 2 * 8 * 4 * 130 * 4
    nbytes, splits, impl = _plan(_desc(Sq=1, Skv=8192, B=2, Hq=8, Hkv=2, D=48, Dv=32, num_splits=4, dtype=capi.F32))
    assert impl == capi.IMPL_SPLITKV_MFMA and splits == 4 and nbytes == 2 * 8 * 4 * 66 * 4
    nbytes, _, impl = _plan(_desc(add_mask=0x20000))                            # dense mask: still the matrix cores, with
    assert impl == capi.IMPL_MFMA and nbytes == 256 + 256                     # 2 x 4 x 4 x 4 block flags and a limit per mask row (each rounded up)
    assert _plan(_desc(add_mask=0x20000, D=80, Dv=80))[2] == capi.IMPL_MFMA
    assert _plan(_desc(add_mask=0x20000, D=160, Dv=160))[2] == capi.IMPL_GENERIC      # (a mask without strides: not readable 8 bytes at a time)
    wide_masked = _desc(add_mask=0x20000, D=160, Dv=160)
    wide_masked.mask_stride[2], wide_masked.mask_stride[3] = 128, 1                    # a [1, 1, Sq, Skv] mask
    nbytes, _, impl = _plan(wide_masked)
    assert impl == capi.IMPL_MFMA and nbytes == 256 + 512                              # block flags and a limit per mask row (128 of them), as at 128
    nbytes, splits, impl = _plan(_desc(Sq=1, Skv=8192, B=32, Hq=32, Hkv=32))
    assert impl == capi.IMPL_SPLITKV_MFMA and splits == 1 and nbytes == 0      # 1024 workgroups, four rounds of 256
    nbytes, splits, impl = _plan(_desc(Sq=1, Skv=2048, B=8, Hq=32, Hkv=32))
    assert impl == capi.IMPL_SPLITKV and splits >= 1                             # one row per KV head, 268 MB of cache: vector ALU
    assert nbytes == (0 if splits == 1 else 8 * 32 * 1 * splits * (128 + 2) * 4)
    # grouped-query decode, 4 rows per KV head: the matrix-core split-KV kernel (the vector-ALU one by name)
    nbytes, splits, impl = _plan(_desc(Sq=1, Skv=8192, B=1, Hq=8, Hkv=2, num_splits=4))
    assert impl == capi.IMPL_SPLITKV_MFMA and splits == 4 and nbytes == 8 * 4 * 130 * 4
    nbytes, splits, impl = _plan(_desc(Sq=1, Skv=8192, B=1, Hq=8, Hkv=2, num_splits=4, impl=capi.IMPL_SPLITKV))
    assert impl == capi.IMPL_SPLITKV and splits == 4 and nbytes == 8 * 4 * 130 * 4
    # its split count fills the device's compute units once (256 here: no device to ask): 2 groups x 128 splits of 64 keys
    # would, but a split keeps at least 256 keys
    _, splits, impl = _plan(_desc(Sq=1, Skv=8192, B=1, Hq=8, Hkv=2))
    assert impl == capi.IMPL_SPLITKV_MFMA and splits == 32
    _, splits, impl = _plan(_desc(Sq=1, Skv=8192, B=32, Hq=32, Hkv=8))
    assert impl == capi.IMPL_SPLITKV_MFMA and splits == 1                     # 256 groups: one round, nothing to combine
    # f32: its own matrix-core split-KV kernel (chunks of 16 or 32 rows) from two rows per KV head on, any number of rows
    assert _plan(_desc(Sq=1, Skv=8192, B=2, Hq=8, Hkv=2, dtype=capi.F32))[2] == capi.IMPL_SPLITKV_MFMA
    assert _plan(_desc(Sq=1, Skv=8192, B=2, Hq=8, Hkv=8, dtype=capi.F32))[2] == capi.IMPL_SPLITKV_MFMA        # one row too, from 512 keys on
    assert _plan(_desc(Sq=1, Skv=400, B=2, Hq=8, Hkv=8, dtype=capi.F32))[2] == capi.IMPL_SPLITKV              # shortest caches: vector ALU
    assert _plan(_desc(Sq=1, Skv=600, B=2, Hq=8, Hkv=8, D=64, Dv=64, dtype=capi.F32))[2] == capi.IMPL_SPLITKV  # (at D = 64 up to 1024 keys)
    assert _plan(_desc(Sq=64, Skv=8192, B=2, Hq=32, Hkv=2, dtype=capi.F32))[2] == capi.IMPL_SPLITKV_MFMA      # 1024 rows per KV head
    assert _plan(_desc(Sq=65, Skv=8192, B=8, Hq=64, Hkv=2, dtype=capi.F32))[2] == capi.IMPL_MFMA              # more positions, 512 row blocks: prefill
    assert _plan(_desc(Sq=1, Skv=100, B=2, Hq=8, Hkv=2, dtype=capi.F32))[2] == capi.IMPL_MFMA                 # shortest caches: one workgroup per head
    _, splits, impl = _plan(_desc(Sq=1, Skv=8192, B=32, Hq=32, Hkv=8, dtype=capi.F32))
    assert impl == capi.IMPL_SPLITKV_MFMA and splits == 1
    assert _plan(_desc(Sq=1, Skv=8192, B=2, Hq=8, Hkv=2, D=64, Dv=64))[2] == capi.IMPL_SPLITKV_MFMA            # D = 64 too
    assert _plan(_desc(Sq=4, Skv=8192, B=2, Hq=32, Hkv=2))[2] == capi.IMPL_SPLITKV_MFMA             # 64 rows per KV head: one workgroup's worth
    _, splits, impl = _plan(_desc(Sq=8, Skv=8192, B=2, Hq=32, Hkv=2))
    assert impl == capi.IMPL_MFMA and splits == 8                                                   # 128 rows per KV head: the prefill kernel, keys split
    assert _plan(_desc(Sq=1, Skv=400, B=2, Hq=4, Hkv=2))[2] == capi.IMPL_SPLITKV                    # 2 rows, short cache: vector ALU
    assert _plan(_desc(Sq=1, Skv=512, B=2, Hq=16, Hkv=2))[2] == capi.IMPL_SPLITKV_MFMA              # 8 rows
    assert _plan(_desc(Sq=1, Skv=8192, B=2, Hq=4, Hkv=2))[2] == capi.IMPL_SPLITKV_MFMA              # 2 rows, long cache
    assert _plan(_desc(Sq=1, Skv=64))[2] in (capi.IMPL_MFMA, capi.IMPL_SPLITKV)
    # long sequences: the same kernel
    def long(**kw):
        S = kw.pop("S", 16384)
        d = _desc(B=4, Hq=32, Hkv=8, Sq=S, Skv=S, **kw)
        for name, heads in (("q_stride", 32), ("k_stride", 8), ("v_stride", 8), ("o_stride", 32)):
            st = getattr(d, name)
            st[0], st[1], st[2] = heads * S * d.D, S * d.D, d.D
        return d
    assert _plan(long())[2] == capi.IMPL_MFMA
    assert _plan(long(causal=1))[2] == capi.IMPL_MFMA
    assert _plan(long(S=4096))[2] == capi.IMPL_MFMA
    assert _plan(long(S=4096, causal=1))[2] == capi.IMPL_MFMA
    assert _plan(long(S=2048))[2] == capi.IMPL_MFMA
    assert _plan(long(D=64, Dv=64))[2] == capi.IMPL_MFMA
    assert _plan(_desc(Sq=8192, Skv=8192))[2] == capi.IMPL_MFMA          # 2 x 4 heads x 32 blocks: too few items
    # few row blocks over many keys: the prefill launch splits the keys (and then needs a workspace for the partial results)
    def chunk(B, Hq, Hkv, Sq, Skv, **kw):
        d = _desc(B=B, Hq=Hq, Hkv=Hkv, Sq=Sq, Skv=Skv, **kw)
        for name, heads, rows in (("q_stride", Hq, Sq), ("k_stride", Hkv, Skv), ("v_stride", Hkv, Skv), ("o_stride", Hq, Sq)):
            st = getattr(d, name)
            st[0], st[1], st[2] = heads * rows * d.D, rows * d.D, d.D
        return d
    nbytes, splits, impl = _plan(chunk(1, 8, 8, 128, 4096, causal=1))
    assert impl == capi.IMPL_MFMA and splits == 4 and nbytes == 1 * 8 * 128 * 4 * 130 * 4       # 8 workgroups, 1024 keys per split at least
    nbytes, splits, impl = _plan(chunk(1, 32, 8, 512, 32768))
    assert impl == capi.IMPL_MFMA and splits == 4                                               # 128 workgroups: 4 x fills both slots of every compute unit
    assert _plan(chunk(1, 32, 8, 512, 32768, num_splits=1))[1] == 1
    assert _plan(chunk(4, 32, 8, 512, 32768))[1] == 1                                           # 512 workgroups: the rows fill the device
    assert _plan(chunk(1, 8, 8, 128, 2048))[1] == 1                                             # too few keys to split
    assert _plan(chunk(1, 8, 8, 4096, 4096, causal=1))[1] == 1                                  # square: the partial results would cost what the splits gain
    assert _plan(chunk(1, 32, 8, 512, 32768, lse=0x30000))[1] == 4                              # (the combine pass writes the row normalisers)
    assert _plan(chunk(1, 32, 8, 512, 32768, dtype=capi.F32))[1] == 4                           # the f32 matrix-core kernel splits the same way
    assert _plan(chunk(1, 32, 8, 512, 32768, add_mask=0x20000))[1] == 1                          # not with a dense mask
    # empty problems need nothing
    assert _plan(_desc(Sq=0))[0] == 0


@pytest.mark.parametrize("kw,code", [
    (dict(dtype=7), capi.EDTYPE),
    (dict(Sq=-1), capi.ESHAPE),
    (dict(Hq=6, Hkv=4), capi.ESHAPE),
    (dict(q=None), capi.EINVAL),
    (dict(impl=9), capi.EINVAL),
    (dict(num_splits=-2), capi.EINVAL),
    (dict(impl=capi.IMPL_MFMA64), capi.EUNSUPPORTED),                 # retired: the value is refused
    (dict(impl=capi.IMPL_MFMA, D=264, Dv=264), capi.EUNSUPPORTED),
    (dict(impl=capi.IMPL_MFMA, D=160, Dv=160, dtype=capi.F32), capi.EUNSUPPORTED),          # above 128 the prefill kernel is 16-bit only
    (dict(impl=capi.IMPL_MFMA, D=84, Dv=84), capi.EUNSUPPORTED),
    (dict(impl=capi.IMPL_SPLITKV, Sq=1, D=96, Dv=96), capi.EUNSUPPORTED),             # the vector-ALU kernel takes 64 and 128 only
    (dict(impl=capi.IMPL_SPLITKV, Sq=4096), capi.EUNSUPPORTED),
    (dict(impl=capi.IMPL_SPLITKV_MFMA, Sq=4096), capi.EUNSUPPORTED),
    (dict(impl=capi.IMPL_SPLITKV_MFMA, Sq=1, D=36, Dv=36), capi.EUNSUPPORTED),
    (dict(impl=capi.IMPL_SPLITKV_MFMA, Sq=1, add_mask=0x20000), capi.EUNSUPPORTED),          # (a mask without a unit key stride)
    (dict(impl=capi.IMPL_SPLITKV_MFMA, Sq=1, add_mask=0x20000, dtype=capi.F32), capi.EUNSUPPORTED),
    (dict(D=512, Dv=512), capi.EUNSUPPORTED),
    (dict(B=70000), capi.ESHAPE),
])
def test_validation_errors(kw, code):
    with pytest.raises(capi.RocmError) as e:
        _plan(_desc(**kw))
    assert e.value.code == code
    assert e.value.message and capi.load().incin_rocm_last_error().decode() == e.value.message


def test_null_descriptor_and_missing_workspace():
    lib = capi.load()
    assert lib.incin_rocm_sdpa_workspace(None, None, None, None) == capi.EINVAL
    assert lib.incin_rocm_sdpa_fwd(None, None) == capi.EINVAL
    d = _desc(Sq=1, Skv=8192, B=1, Hq=8, Hkv=8, num_splits=4)
    with pytest.raises(capi.RocmError) as e:      # rejected before any device is touched
        capi.sdpa_fwd(d)
    assert e.value.code == capi.EWORKSPACE
    assert lib.incin_rocm_device_count(None) == capi.EINVAL


def test_mask_row_limits_validation():
    """incin_rocm_mask_row_limits refuses what it cannot read before it touches a device."""
    lib = capi.load()
    shape = (C.c_int64 * 4)(1, 1, 8, 16)
    strides = (C.c_int64 * 4)(0, 0, 16, 1)
    assert lib.incin_rocm_mask_row_limits(0, 7, 0x1000, shape, strides, 0x2000, None) == capi.EDTYPE
    assert lib.incin_rocm_mask_row_limits(0, capi.F32, 0x1000, None, strides, 0x2000, None) == capi.EINVAL
    assert lib.incin_rocm_mask_row_limits(0, capi.F32, 0x1000, (C.c_int64 * 4)(1, -1, 8, 16), strides, 0x2000, None) == capi.ESHAPE
    assert lib.incin_rocm_mask_row_limits(0, capi.F32, 0x1000, shape, strides, None, None) == capi.EINVAL
    assert lib.incin_rocm_mask_row_limits(0, capi.F32, None, (C.c_int64 * 4)(1, 1, 0, 16), strides, None, None) == 0      # no rows: nothing to do


def test_matrix_rate_validation():
    # the diagnostic refuses malformed requests before any device is touched
    import ctypes as C
    lib = capi.load()
    fl = C.c_double(0.0)
    assert lib.incin_rocm_matrix_rate(0, None, 0x1000, 0, 10, C.byref(fl), None) == capi.EINVAL
    assert lib.incin_rocm_matrix_rate(0, 0x1000, 0x1000, 0, 10, None, None) == capi.EINVAL
    assert lib.incin_rocm_matrix_rate(0, 0x1000, 0x1000, 2, 10, C.byref(fl), None) == capi.EINVAL
    assert lib.incin_rocm_matrix_rate(0, 0x1000, 0x1000, 0, 0, C.byref(fl), None) == capi.EINVAL
    assert b"matrix_rate" in lib.incin_rocm_last_error()
    # and so does the read-rate one
    assert lib.incin_rocm_read_rate(0, None, 1 << 27, 1, 0x1000, None) == capi.EINVAL
    assert lib.incin_rocm_read_rate(0, 0x1000, 1 << 27, 1, None, None) == capi.EINVAL
    assert lib.incin_rocm_read_rate(0, 0x1000, 0, 1, 0x1000, None) == capi.EINVAL
    assert lib.incin_rocm_read_rate(0, 0x1000, (1 << 27) + 4096, 1, 0x1000, None) == capi.EINVAL      # not a multiple of 128 MiB
    assert lib.incin_rocm_read_rate(0, 0x1008, 1 << 27, 1, 0x1000, None) == capi.EINVAL               # misaligned
    assert b"read_rate" in lib.incin_rocm_last_error()
    assert lib.incin_rocm_lds_fill(0, 0x7fc00000, None, None) == capi.EINVAL
    assert b"lds_fill" in lib.incin_rocm_last_error()


def _bwd(fwd_kw=None, **kw):
    bd = capi.SdpaBwdDesc()
    bd.fwd = _desc(**{**dict(lse=0x30000), **(fwd_kw or {})})
    for name, heads in (("d_o", 4), ("d_q", 4), ("d_k", 4), ("d_v", 4)):
        setattr(bd, name, 0x40000)
        st = getattr(bd, name + "_stride")
        st[0], st[1], st[2] = heads * 128 * 128, 128 * 128, 128
    for k, v in kw.items():
        setattr(bd, k, v)
    return bd


def test_backward_validation_and_workspace_size():
    # two f32 per query row, whichever kernels take the request
    assert capi.sdpa_bwd_workspace(_bwd()) == 2 * 2 * 4 * 128 * 4
    assert capi.sdpa_bwd_workspace(_bwd(dict(dtype=capi.F32))) == 2 * 2 * 4 * 128 * 4
    # ... plus, for a dense mask on the matrix-core kernels, the mask's block flags (a byte per 32 rows x 32 keys, in 256s)
    assert capi.sdpa_bwd_workspace(_bwd(dict(add_mask=0x20000))) == 2 * 2 * 4 * 128 * 4 + 256
    assert capi.sdpa_bwd_workspace(_bwd(dict(add_mask=0x20000, mask_stride=(4 * 128 * 128, 128 * 128, 128, 1)))) == 2 * 2 * 4 * 128 * 4 + 256      # 8 mask planes x 16 flags, rounded up
    assert capi.sdpa_bwd_workspace(_bwd(dict(add_mask=0x20000, impl=capi.IMPL_GENERIC))) == 2 * 2 * 4 * 128 * 4
    assert capi.sdpa_bwd_workspace(_bwd(dict(add_mask=0x20000, dtype=capi.F32))) == 2 * 2 * 4 * 128 * 4 + 256
    assert capi.sdpa_bwd_workspace(_bwd(dict(Sq=0))) == 0            # nothing to compute
    # ... plus, for an f32 call on the matrix-core kernels that does not fill the device, the planes that the parts of a
    # block sum into: 2 x 4 heads x 1024 rows are 64 blocks of 128 for either kernel, a quarter of the 256 workgroups a device
    # of 256 compute units (no device to ask here) holds at D = 128 - four parts, three planes per gradient
    def long(S=1024, **fwd_kw):
        bd = _bwd(dict(Sq=S, Skv=S, **fwd_kw))
        for st in (bd.fwd.q_stride, bd.fwd.k_stride, bd.fwd.v_stride, bd.fwd.o_stride, bd.d_o_stride, bd.d_q_stride, bd.d_k_stride, bd.d_v_stride):
            st[0], st[1], st[2] = 4 * S * 128, S * 128, 128
        return bd
    rows, plane = 2 * 2 * 4 * 1024 * 4, 2 * 4 * 1024 * 128 * 4
    assert capi.sdpa_bwd_workspace(long()) == rows                                          # (16-bit storage: walks of 16 tiles are not dealt)
    # 16-bit storage, four query heads on one KV head x 4096 keys: 64 key blocks whose walks of 256 tiles go to four workgroups
    # each, every one with a plane for dK and one for dV
    assert capi.sdpa_bwd_workspace(long(S=4096, Hkv=1)) == 4 * rows + 4 * 2 * (2 * 4096 * 128 * 4)
    assert capi.sdpa_bwd_workspace(long(S=4096, Hkv=1, B=8)) == 16 * rows                    # (a full round of key blocks: not dealt)
    assert capi.sdpa_bwd_workspace(long(dtype=capi.F32)) == rows + 3 * 3 * plane
    assert capi.sdpa_bwd_workspace(long(dtype=capi.F32, impl=capi.IMPL_GENERIC)) == rows
    assert capi.sdpa_bwd_workspace(long(dtype=capi.F32, D=64, Dv=64)) == rows + 3 * 3 * plane // 2      # (512 workgroups at a time at D = 64)
    assert capi.sdpa_bwd_workspace(long(dtype=capi.F32, B=8)) == 4 * rows                     # a full round of blocks: not dealt
    assert capi.sdpa_bwd_workspace(long(dtype=capi.F32, B=4)) == 2 * rows + 3 * 2 * plane     # half a round: two parts
    for bd, code in [
        (_bwd(dict(lse=None)), capi.EINVAL),                          # the forward's normalisers are an input
        (_bwd(d_k=None), capi.EINVAL),
        (_bwd(dict(impl=capi.IMPL_MFMA, D=160, Dv=160)), capi.EUNSUPPORTED),         # pinned to kernels that do not take it
        (_bwd(dict(impl=capi.IMPL_MFMA, D=36, Dv=36)), capi.EUNSUPPORTED),           # (72-byte rows are not whole vectors)
        (_bwd(dict(impl=capi.IMPL_MFMA, dtype=capi.F32, D=160, Dv=160)), capi.EUNSUPPORTED),
        (_bwd(dict(impl=capi.IMPL_MFMA, add_mask=0x20000, mask_stride=(0, 0, 1 << 25, 1))), capi.EUNSUPPORTED),      # (64 rows of the mask do not fit 32-bit offsets)
        (_bwd(dict(impl=capi.IMPL_SPLITKV)), capi.EUNSUPPORTED),
        (_bwd(dict(D=320, Dv=320)), capi.EUNSUPPORTED),
        (_bwd(dict(Hq=6, Hkv=4)), capi.ESHAPE),
    ]:
        with pytest.raises(capi.RocmError) as e:
            capi.sdpa_bwd_workspace(bd)
        assert e.value.code == code, e.value.message
    lib = capi.load()
    assert lib.incin_rocm_sdpa_bwd(None, None) == capi.EINVAL
    with pytest.raises(capi.RocmError) as e:          # no workspace: rejected before any device is touched
        capi.sdpa_bwd(_bwd())
    assert e.value.code == capi.EWORKSPACE
