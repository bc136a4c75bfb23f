"""numpy-facing driver of the C ABI: upload, describe, launch, download.

This is test/benchmark plumbing around `incin_rocm_sdpa_fwd` for 4-D
[B, H, S, D] operands; the rank-generic operator mirror lives in the C++ host
layer (incin_amd/host/).  Everything computed comes from the GPU library.
"""
import ctypes as C
import math

import numpy as np

from . import capi, dtypes


def _strides3(arr_shape, bcast_b=False, bcast_h=False):
    _, h, s, d = arr_shape
    return (0 if bcast_b else h * s * d, 0 if bcast_h else s * d, d)


class DeviceTensor:
    """A contiguous [B, H, S, D] tensor in device memory."""

    def __init__(self, shape, dtype, dev=0, buf=None):
        self.shape = tuple(int(x) for x in shape)
        self.dtype = dtype
        self.dev = dev
        n = int(np.prod(self.shape)) if len(self.shape) else 1
        self.buf = buf if buf is not None else capi.DeviceBuffer(n * dtypes.ITEMSIZE[dtype], dev)

    @classmethod
    def from_f32(cls, x, dtype, dev=0):
        raw = dtypes.encode(x, dtype)
        return cls(raw.shape, dtype, dev, capi.DeviceBuffer.from_numpy(raw, dev))

    def to_f32(self):
        raw = self.buf.to_numpy(dtypes.storage_numpy_dtype(self.dtype), self.shape)
        return dtypes.decode(raw, self.dtype)

    @property
    def ptr(self):
        return self.buf.ptr


def resolve_scale(scale, d):
    """(float) scale.unwrap_or(1/sqrt(D)): shape_ops.rs:1259-1261 then elementwise_kernel.rs:87."""
    s = (1.0 / math.sqrt(float(d))) if scale is None else float(scale)
    return float(np.float32(s))


def make_desc(q, k, v, o, scale=None, causal=False, kv_lens=None, mask=None, mask_strides=None,
              num_splits=0, impl=capi.IMPL_AUTO, workspace=None, q_lens=None, lse=None):
    B, Hq, Sq, D = q.shape
    Bk, Hkv, Skv, Dk = k.shape
    Bv, Hv, Skv2, Dv = v.shape
    d = capi.SdpaDesc()
    d.dtype, d.device = q.dtype, q.dev
    d.B, d.Hq, d.Hkv, d.Sq, d.Skv, d.D, d.Dv = B, Hq, Hkv, Sq, Skv, D, Dv
    for name, t in (("q_stride", q), ("k_stride", k), ("v_stride", v), ("o_stride", o)):
        st = _strides3(t.shape, bcast_b=(t.shape[0] == 1 and B > 1))
        for i in range(3):
            getattr(d, name)[i] = st[i]
    d.q, d.k, d.v, d.o = q.ptr, k.ptr, v.ptr, o.ptr
    d.scale = resolve_scale(scale, D)
    d.causal = 1 if causal else 0
    d.kv_lens = kv_lens.ptr if kv_lens is not None else None
    d.q_lens = q_lens.ptr if q_lens is not None else None
    d.lse = lse.ptr if lse is not None else None
    if mask is not None:
        d.add_mask = mask.ptr
        for i in range(4):
            d.mask_stride[i] = mask_strides[i]
    d.num_splits = num_splits
    d.impl = impl
    if workspace is not None:
        d.workspace, d.workspace_bytes = workspace.ptr, workspace.nbytes
    return d


def mask_strides_for(mask_shape, B, Hq, Sq, Skv):
    """Element strides (batch, head, row, key) of a contiguous mask broadcastable to [B,Hq,Sq,Skv]."""
    shp = [1] * (4 - len(mask_shape)) + list(mask_shape)
    full = [B, Hq, Sq, Skv]
    st, acc = [0] * 4, 1
    for a in range(3, -1, -1):
        if shp[a] not in (1, full[a]):
            raise ValueError("mask shape %r does not broadcast to %r" % (tuple(mask_shape), tuple(full)))
        st[a] = 0 if (shp[a] == 1 and full[a] != 1) else acc
        acc *= shp[a]
    return st


def sdpa(q, k, v, dtype=capi.F32, scale=None, causal=False, kv_lens=None, mask=None,
         num_splits=0, impl=capi.IMPL_AUTO, dev=0, return_info=False, q_lens=None, return_lse=False, mask_row_pitch=None):
    """Run attention on the GPU for f32 numpy operands [B,Hq,Sq,D], [B,Hkv,Skv,D], [B,Hkv,Skv,Dv].

    Operands are rounded to `dtype` on upload; the result is returned as f32
    holding the `dtype`-rounded output.  `mask_row_pitch`: the mask's rows are stored that many elements apart
    (a view of a wider buffer whose padding holds a large value no kernel may read as a key's).
    """
    q = np.asarray(q, dtype=np.float32)
    k = np.asarray(k, dtype=np.float32)
    v = np.asarray(v, dtype=np.float32)
    B, Hq, Sq, D = q.shape
    Dv = v.shape[-1]
    tq, tk, tv = (DeviceTensor.from_f32(x, dtype, dev) for x in (q, k, v))
    to = DeviceTensor((B, Hq, Sq, Dv), dtype, dev)
    tl = capi.DeviceBuffer.from_numpy(np.asarray(kv_lens, dtype=np.int32), dev) if kv_lens is not None else None
    tql = capi.DeviceBuffer.from_numpy(np.asarray(q_lens, dtype=np.int32), dev) if q_lens is not None else None
    tm, ms = None, None
    if mask is not None:
        mask = np.asarray(mask, dtype=np.float32)
        if mask_row_pitch is not None:
            padded = np.full(mask.shape[:-1] + (mask_row_pitch,), 1e4, np.float32)
            padded[..., :mask.shape[-1]] = mask
            ms = mask_strides_for(mask.shape[:-1] + (k.shape[2],), B, Hq, Sq, k.shape[2])
            ms = [st // k.shape[2] * mask_row_pitch for st in ms[:3]] + [ms[3]]
            mask = padded
        else:
            ms = mask_strides_for(mask.shape, B, Hq, Sq, k.shape[2])
        tm = capi.DeviceBuffer.from_numpy(dtypes.encode(mask, dtype), dev)
    tlse = capi.DeviceBuffer(B * Hq * Sq * 4, dev) if return_lse else None
    d = make_desc(tq, tk, tv, to, scale, causal, tl, tm, ms, num_splits, impl, q_lens=tql, lse=tlse)
    nbytes, splits, chosen = capi.sdpa_workspace(d)
    ws = capi.DeviceBuffer(nbytes, dev) if nbytes else None
    if ws is not None:
        d.workspace, d.workspace_bytes = ws.ptr, ws.nbytes
    capi.sdpa_fwd(d)
    capi.sync(dev)
    out = to.to_f32()
    lse = tlse.to_numpy(np.float32, (B, Hq, Sq)) if return_lse else None
    for t in (tq.buf, tk.buf, tv.buf, to.buf, tl, tm, ws, tql, tlse):
        if t is not None:
            t.free()
    info = {"impl": chosen, "splits": splits, "workspace_bytes": nbytes}
    if return_lse:
        return (out, lse, info) if return_info else (out, lse)
    if return_info:
        return out, info
    return out


def sdpa_backward(q, k, v, d_out, dtype=capi.BF16, scale=None, causal=False, kv_lens=None, impl=capi.IMPL_AUTO, dev=0, mask=None,
                  q_lens=None, poison_padding=False):
    """Forward (with row normalisers) then backward on the GPU for f32 numpy operands [B,Hq,Sq,D], [B,Hkv,Skv,D],
    [B,Hkv,Skv,Dv], d_out [B,Hq,Sq,Dv] and an optional dense additive mask broadcastable to [B,Hq,Sq,Skv]; returns
    (out, dq, dk, dv) as f32 holding the `dtype`-rounded results.  `impl` pins the kernels of both passes.  q_lens: query
    rows at and beyond are padding; poison_padding overwrites what the forward left in their O and lse rows with NaN
    bit patterns before the backward runs (it must not read them)."""
    q, k, v, d_out = (np.asarray(x, dtype=np.float32) for x in (q, k, v, d_out))
    B, Hq, Sq, D = q.shape
    Dv = v.shape[-1]
    tq, tk, tv, tg = (DeviceTensor.from_f32(x, dtype, dev) for x in (q, k, v, d_out))
    to, tdq = DeviceTensor((B, Hq, Sq, Dv), dtype, dev), DeviceTensor(q.shape, dtype, dev)
    tdk, tdv = DeviceTensor(k.shape, dtype, dev), DeviceTensor(v.shape, dtype, dev)
    tl = capi.DeviceBuffer.from_numpy(np.asarray(kv_lens, dtype=np.int32), dev) if kv_lens is not None else None
    tm, ms = None, None
    if mask is not None:
        mask = np.asarray(mask, dtype=np.float32)
        ms = mask_strides_for(mask.shape, B, Hq, Sq, k.shape[2])
        tm = capi.DeviceBuffer.from_numpy(dtypes.encode(mask, dtype), dev)
    tql = capi.DeviceBuffer.from_numpy(np.asarray(q_lens, dtype=np.int32), dev) if q_lens is not None else None
    tlse = capi.DeviceBuffer(max(B * Hq * Sq, 1) * 4, dev)
    bd = capi.SdpaBwdDesc()
    bd.fwd = make_desc(tq, tk, tv, to, scale, causal, tl, tm, ms, impl=impl, lse=tlse, q_lens=tql)
    fbytes = capi.sdpa_workspace(bd.fwd)[0]
    fws = capi.DeviceBuffer(fbytes, dev) if fbytes else None
    if fws is not None:
        bd.fwd.workspace, bd.fwd.workspace_bytes = fws.ptr, fws.nbytes
    capi.sdpa_fwd(bd.fwd)
    if poison_padding and q_lens is not None:
        capi.sync(dev)
        o_host, l_host = to.to_f32(), tlse.to_numpy(np.float32, (B, Hq, Sq))
        for b in range(B):
            o_host[b, :, int(q_lens[b]):] = np.nan
            l_host[b, :, int(q_lens[b]):] = np.nan
        raw = dtypes.encode(o_host, dtype)
        capi.check(capi.load().incin_rocm_memcpy_h2d(dev, to.ptr, raw.ctypes.data, raw.nbytes))
        capi.check(capi.load().incin_rocm_memcpy_h2d(dev, tlse.ptr, l_host.ctypes.data, l_host.nbytes))
    for name, t in (("d_o", tg), ("d_q", tdq), ("d_k", tdk), ("d_v", tdv)):
        setattr(bd, name, t.ptr)
        st = _strides3(t.shape)
        for i in range(3):
            getattr(bd, name + "_stride")[i] = st[i]
    nbytes = capi.sdpa_bwd_workspace(bd)
    ws = capi.DeviceBuffer(nbytes, dev) if nbytes else None
    if ws is not None:
        bd.workspace, bd.workspace_bytes = ws.ptr, ws.nbytes
    capi.sdpa_bwd(bd)
    capi.sync(dev)
    res = tuple(t.to_f32() for t in (to, tdq, tdk, tdv))
    for t in (tq.buf, tk.buf, tv.buf, tg.buf, to.buf, tdq.buf, tdk.buf, tdv.buf, tl, tm, tlse, ws, fws, tql):
        if t is not None:
            t.free()
    return res
