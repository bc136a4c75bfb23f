"""TEST INFRASTRUCTURE ONLY -- numpy-facing loader for the CPU oracle.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import
this module; the product (``incin_amd``) never does.

``sdpa``            the reference CPU op's arithmetic (C restatement, row-streaming form)
``sdpa_rows``       the same for selected (batch, query-row) pairs
``sdpa_materialised`` the same laid out as the reference executes it (CPU-baseline timing)
``brute_f64``       an independent float64 numpy evaluation of softmax(q k^T s + m) v

Shapes follow the reference operator (crates/incin-core/src/tensor/backend.rs:485-492):
q ``[..., Sq, D]``, k ``[..., Skv, D]``, v ``[..., Skv, Dv]``, mask broadcastable to
``[..., Sq, Skv]``; leading axes broadcast NumPy-style
(crates/incin-backends/src/cpu/ops/matmul.rs:198-221, cpu/stride.rs:86-106).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
MAXB = 6


def build(force=False):
    """Compile liboracle.so with the committed Makefile."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


class _Desc(C.Structure):
    _fields_ = [
        ("nb", C.c_int32),
        ("bshape", C.c_int64 * MAXB),
        ("q_bs", C.c_int64 * MAXB),
        ("k_bs", C.c_int64 * MAXB),
        ("v_bs", C.c_int64 * MAXB),
        ("m_bs", C.c_int64 * MAXB),
        ("Sq", C.c_int64), ("Skv", C.c_int64), ("D", C.c_int64), ("Dv", C.c_int64),
        ("q_rs", C.c_int64), ("q_cs", C.c_int64),
        ("k_rs", C.c_int64), ("k_cs", C.c_int64),
        ("v_rs", C.c_int64), ("v_cs", C.c_int64),
        ("m_rs", C.c_int64), ("m_cs", C.c_int64),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p),
        ("mask", C.c_void_p),
        ("causal", C.c_int32),
        ("kv_lens", C.c_void_p),
        ("kv_lens_bs", C.c_int64 * MAXB),
        ("has_scale", C.c_int32),
        ("scale", C.c_double),
        ("host_has_fma", C.c_int32),
    ]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.oracle_struct_size.restype = C.c_size_t
        assert _lib.oracle_struct_size() == C.sizeof(_Desc), "oracle struct layout drifted"
        _lib.oracle_batch_count.restype = C.c_int64
        for name in ("oracle_sdpa", "oracle_sdpa_materialised", "oracle_sdpa_rows"):
            getattr(_lib, name).restype = C.c_int
    return _lib


def broadcast_shape(a, b):
    """Right-aligned NumPy rule, as cpu/stride.rs:86-106 states it."""
    n = max(len(a), len(b))
    out = []
    for i in range(n):
        da = a[len(a) - n + i] if len(a) - n + i >= 0 else 1
        db = b[len(b) - n + i] if len(b) - n + i >= 0 else 1
        if da != db and da != 1 and db != 1:
            raise ValueError(f"cannot broadcast shapes {tuple(a)} and {tuple(b)}")
        out.append(max(da, db))
    return out


def _elem_strides(x):
    return [s // x.itemsize for s in x.strides]


def _aligned_batch_strides(x, ntrail, bshape):
    """Strides (elements) of x's leading axes, right-aligned to bshape; 0 where broadcast."""
    nb = len(bshape)
    lead_shape = list(x.shape[: x.ndim - ntrail])
    lead_str = _elem_strides(x)[: x.ndim - ntrail]
    out = [0] * nb
    for a in range(len(lead_shape)):
        tgt = nb - len(lead_shape) + a
        out[tgt] = 0 if lead_shape[a] == 1 else lead_str[a]
    return out


def _prepare(q, k, v, mask, scale, causal, kv_lens, host_has_fma):
    q = np.asarray(q, dtype=np.float32)
    k = np.asarray(k, dtype=np.float32)
    v = np.asarray(v, dtype=np.float32)
    if q.ndim < 2 or k.ndim < 2 or v.ndim < 2:
        raise ValueError("rank >= 2 required")
    Sq, D = q.shape[-2:]
    Skv, Dk = k.shape[-2:]
    Skv2, Dv = v.shape[-2:]
    if D != Dk or Skv != Skv2:
        raise ValueError("inner dims must match")
    b = broadcast_shape(q.shape[:-2], k.shape[:-2])
    b = broadcast_shape(b, v.shape[:-2])
    if mask is not None and (causal or kv_lens is not None):
        # the reference knows one mask tensor; the synthesised forms stand in for it, they do not add to it
        raise ValueError("give either an explicit mask or causal / kv_lens; fold them into the mask to combine them")
    if mask is not None:
        mask = np.asarray(mask, dtype=np.float32)
        mshape = list(mask.shape)
        while len(mshape) < 2:
            mshape.insert(0, 1)
        mask = mask.reshape(mshape)
        if Sq == 1 and mshape[-2] > 1:
            # the reference's add broadcasts both ways (shape_ops.rs:1262-1266, cpu/stride.rs:86-106): scores [.., 1, Skv]
            # plus a mask of R rows are R rows of scores, each from q's one row - a stride-0 view of q says the same
            Sq = mshape[-2]
            q = np.broadcast_to(q, q.shape[:-2] + (Sq, D))
        if broadcast_shape(mshape[-2:], [Sq, Skv]) != [Sq, Skv]:
            raise ValueError("mask must broadcast to [..., Sq, Skv]")
        b = broadcast_shape(b, mshape[:-2])
    if len(b) > MAXB:
        raise ValueError("too many batch axes")
    d = _Desc()
    d.nb = len(b)
    for i, s in enumerate(b):
        d.bshape[i] = s
    for name, arr in (("q_bs", q), ("k_bs", k), ("v_bs", v)):
        st = _aligned_batch_strides(arr, 2, b)
        for i, s in enumerate(st):
            getattr(d, name)[i] = s
    d.Sq, d.Skv, d.D, d.Dv = Sq, Skv, D, Dv
    qs, ks, vs = _elem_strides(q), _elem_strides(k), _elem_strides(v)
    d.q_rs, d.q_cs = qs[-2], qs[-1]
    d.k_rs, d.k_cs = ks[-2], ks[-1]
    d.v_rs, d.v_cs = vs[-2], vs[-1]
    d.q, d.k, d.v = q.ctypes.data, k.ctypes.data, v.ctypes.data
    keep = [q, k, v]
    if mask is not None:
        st = _aligned_batch_strides(mask, 2, b)
        for i, s in enumerate(st):
            d.m_bs[i] = s
        ms = _elem_strides(mask)
        d.m_rs = 0 if mask.shape[-2] == 1 else ms[-2]
        d.m_cs = 0 if mask.shape[-1] == 1 else ms[-1]
        d.mask = mask.ctypes.data
        keep.append(mask)
    d.causal = 1 if causal else 0
    if kv_lens is not None:
        kv_lens = np.ascontiguousarray(kv_lens, dtype=np.int32)
        st = _aligned_batch_strides(kv_lens, 0, b)
        for i, s in enumerate(st):
            d.kv_lens_bs[i] = s
        d.kv_lens = kv_lens.ctypes.data
        keep.append(kv_lens)
    d.has_scale = 0 if scale is None else 1
    d.scale = 0.0 if scale is None else float(scale)
    d.host_has_fma = 1 if host_has_fma else 0
    return d, b, keep


def sdpa(q, k, v, mask=None, scale=None, causal=False, kv_lens=None, host_has_fma=True):
    """Reference CPU attention op, f32, output [..., Sq, Dv].

    ``causal``/``kv_lens`` synthesise the additive 0/-inf mask the reference's own
    ops would build (``full(-inf).triu(1)``; shape_ops.rs:808-830) without
    materialising it; ``kv_lens`` has the batch shape (broadcastable) and masks
    keys ``j >= len``.
    """
    d, b, keep = _prepare(q, k, v, mask, scale, causal, kv_lens, host_has_fma)
    out = np.empty(list(b) + [d.Sq, d.Dv], dtype=np.float32)
    if out.size:
        rc = lib().oracle_sdpa(C.byref(d), C.c_void_p(out.ctypes.data))
        if rc:
            raise MemoryError("oracle_sdpa")
    del keep
    return out


def sdpa_materialised(q, k, v, mask=None, scale=None, causal=False, kv_lens=None, host_has_fma=True):
    d, b, keep = _prepare(q, k, v, mask, scale, causal, kv_lens, host_has_fma)
    out = np.empty(list(b) + [d.Sq, d.Dv], dtype=np.float32)
    if out.size:
        rc = lib().oracle_sdpa_materialised(C.byref(d), C.c_void_p(out.ctypes.data))
        if rc:
            raise MemoryError("oracle_sdpa_materialised")
    del keep
    return out


def sdpa_rows(q, k, v, rows, mask=None, scale=None, causal=False, kv_lens=None, host_has_fma=True):
    """Selected rows.  ``rows`` is an int array [n, 2] of (flat batch index over the
    broadcast batch shape, query index); returns [n, Dv]."""
    d, b, keep = _prepare(q, k, v, mask, scale, causal, kv_lens, host_has_fma)
    rows = np.asarray(rows, dtype=np.int64).reshape(-1, 2)
    rb = np.ascontiguousarray(rows[:, 0])
    ri = np.ascontiguousarray(rows[:, 1])
    out = np.empty((rows.shape[0], d.Dv), dtype=np.float32)
    if rows.shape[0]:
        rc = lib().oracle_sdpa_rows(C.byref(d), C.c_int64(rows.shape[0]), C.c_void_p(rb.ctypes.data),
                                    C.c_void_p(ri.ctypes.data), C.c_void_p(out.ctypes.data))
        if rc:
            raise MemoryError("oracle_sdpa_rows")
    del keep
    return out


def gemm(lhs, rhs, host_has_fma=True):
    """2-D matmul through the reference's kernel choice (matmul.rs:316-329)."""
    lhs = np.asarray(lhs, dtype=np.float32)
    rhs = np.asarray(rhs, dtype=np.float32)
    m, kk = lhs.shape
    k2, n = rhs.shape
    assert kk == k2
    out = np.empty((m, n), dtype=np.float32)
    ls, rs = _elem_strides(lhs), _elem_strides(rhs)
    lib().oracle_gemm(C.c_int64(m), C.c_int64(kk), C.c_int64(n),
                      C.c_void_p(lhs.ctypes.data), C.c_int64(ls[0]), C.c_int64(ls[1]),
                      C.c_void_p(rhs.ctypes.data), C.c_int64(rs[0]), C.c_int64(rs[1]),
                      C.c_void_p(out.ctypes.data), C.c_int(1 if host_has_fma else 0))
    return out


def softmax_lastdim(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    flat = x.reshape(-1, x.shape[-1])
    out = np.empty_like(flat)
    tmp = np.empty(x.shape[-1], dtype=np.float32)
    for r in range(flat.shape[0]):
        lib().oracle_softmax_row(C.c_void_p(flat[r].ctypes.data), C.c_int64(flat.shape[1]),
                                 C.c_void_p(out[r].ctypes.data), C.c_void_p(tmp.ctypes.data))
    return out.reshape(x.shape)


def log_softmax_lastdim(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    flat = x.reshape(-1, x.shape[-1])
    out = np.empty_like(flat)
    for r in range(flat.shape[0]):
        lib().oracle_log_softmax_row(C.c_void_p(flat[r].ctypes.data), C.c_int64(flat.shape[1]),
                                     C.c_void_p(out[r].ctypes.data))
    return out.reshape(x.shape)


def triu(x, k):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    lib().oracle_triu(C.c_void_p(x.ctypes.data), C.c_int64(x.shape[0]), C.c_int64(x.shape[1]),
                      C.c_int64(k), C.c_void_p(out.ctypes.data))
    return out


def causal_additive_mask(sq, skv):
    """The reference-ops construction of a causal mask: full(-inf,[Sq,Skv]).triu(1 + Skv - Sq)."""
    return triu(np.full((sq, skv), -np.inf, dtype=np.float32), 1 + skv - sq)


def brute_f64(q, k, v, mask=None, scale=None):
    """Independent float64 evaluation; shares no code with the C restatement."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    s = (1.0 / np.sqrt(q.shape[-1])) if scale is None else float(scale)
    x = np.matmul(q, np.swapaxes(k, -1, -2)) * s
    if mask is not None:
        x = x + np.asarray(mask, dtype=np.float64)
    with np.errstate(invalid="ignore"):
        x = x - np.max(x, axis=-1, keepdims=True)
        e = np.exp(x)
        p = e / np.sum(e, axis=-1, keepdims=True)
    return np.matmul(p, v)
