"""ctypes view of the C++ host mirror (incin_amd/host/rocm_backend.hpp).

`RocmStorage` objects stand where the reference's backend storages stand and
`scaled_dot_product_attention` takes the reference's arguments: q, k, v,
optional additive mask, optional scale (incin-core/src/tensor/backend.rs:485-492).
Failures raise `BackendError` whose `.kind` names the incin_core::Error variant
(incin-core/src/err.rs:109-223).  All logic lives in the C++ library; this file
only converts numpy arrays to bytes and back.
"""
import ctypes as C
import os

import numpy as np

from . import dtypes as DT

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("INCIN_ROCM_HOST_LIBRARY") or os.path.join(_HERE, "lib", "libincin_rocm_host.so")

F32, F16, BF16 = 0, 1, 2
KINDS = ["None", "Msg", "ShapeMismatch", "DTypeStorageMismatch", "DeviceMismatch", "UnsupportedDType",
         "InvalidDeviceOrdinal", "OutOfMemory", "UnsupportedBackendOperation"]
EXPORTS = [
    "incin_host_last_error", "incin_host_from_bytes", "incin_host_numel", "incin_host_rank", "incin_host_shape", "incin_host_strides",
    "incin_host_dtype", "incin_host_to_bytes", "incin_host_transpose", "incin_host_broadcast_as",
    "incin_host_narrow", "incin_host_tag_causal", "incin_host_tag_key_padding", "incin_host_infer_mask_tag",
    "incin_host_scaled_dot_product_attention", "incin_host_attention_backward", "incin_host_release", "incin_host_last_launch_count",
    "incin_host_capability_name", "incin_host_capability_max_rank", "incin_host_capability_support",
    "incin_host_capability_rule_count", "incin_host_capability_rule", "incin_host_capability_docs",
    "incin_host_lower_attention", "incin_host_attention_spec_out_dims", "incin_host_execute_attention",
    "incin_host_release_attention_spec", "incin_host_reshape",
    "incin_host_is_compiled_in", "incin_host_probe", "incin_host_detect_device",
    "incin_host_data_ptr", "incin_host_set_stream", "incin_host_begin_recording", "incin_host_end_recording", "incin_host_replay",
    "incin_host_release_graph", "incin_host_pool_stats", "incin_host_trim_pool",
]


class BackendError(RuntimeError):
    def __init__(self, code, message):
        self.kind = KINDS[code] if 0 <= code < len(KINDS) else "Unknown(%d)" % code
        self.message = message
        super().__init__("%s: %s" % (self.kind, message))


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError("%s is not built; run `python -m incin_amd.build`" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        L.incin_host_last_error.restype = C.c_char_p
        L.incin_host_last_launch_count.restype = C.c_int64
        L.incin_host_release.restype = None
        L.incin_host_release.argtypes = [C.c_void_p]
        L.incin_host_from_bytes.argtypes = [C.c_void_p, C.c_size_t, C.POINTER(C.c_int64), C.c_int32, C.c_int32, C.c_int32,
                                            C.POINTER(C.c_void_p)]
        L.incin_host_numel.argtypes = [C.c_void_p, C.POINTER(C.c_int64)]
        L.incin_host_rank.argtypes = [C.c_void_p, C.POINTER(C.c_int32)]
        L.incin_host_shape.argtypes = [C.c_void_p, C.POINTER(C.c_int64)]
        L.incin_host_strides.argtypes = [C.c_void_p, C.POINTER(C.c_int64)]
        L.incin_host_dtype.argtypes = [C.c_void_p, C.POINTER(C.c_int32)]
        L.incin_host_to_bytes.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.incin_host_transpose.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.POINTER(C.c_void_p)]
        L.incin_host_broadcast_as.argtypes = [C.c_void_p, C.POINTER(C.c_int64), C.c_int32, C.POINTER(C.c_void_p)]
        L.incin_host_narrow.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.POINTER(C.c_void_p)]
        L.incin_host_tag_causal.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        L.incin_host_tag_key_padding.argtypes = [C.c_void_p, C.POINTER(C.c_int32), C.c_int64, C.POINTER(C.c_void_p)]
        L.incin_host_infer_mask_tag.argtypes = [C.c_void_p, C.POINTER(C.c_int32), C.POINTER(C.c_void_p)]
        L.incin_host_scaled_dot_product_attention.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32,
                                                              C.c_double, C.POINTER(C.c_void_p)]
        L.incin_host_attention_backward.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_double, C.c_void_p] + \
                                                   [C.POINTER(C.c_void_p)] * 4
        L.incin_host_capability_name.restype = C.c_char_p
        L.incin_host_capability_name.argtypes = [C.c_int32, C.c_int32]
        L.incin_host_capability_max_rank.restype = C.c_int32
        L.incin_host_capability_support.argtypes = [C.c_int32] * 7 + [C.POINTER(C.c_int32), C.c_char_p, C.c_size_t]
        L.incin_host_capability_rule_count.restype = C.c_int32
        L.incin_host_capability_rule_count.argtypes = [C.c_int32]
        L.incin_host_capability_rule.argtypes = [C.c_int32, C.c_int32, C.POINTER(C.c_int32), C.POINTER(C.c_uint32),
                                                 C.POINTER(C.c_uint32), C.POINTER(C.c_int32), C.POINTER(C.c_int32),
                                                 C.POINTER(C.c_int32), C.POINTER(C.c_uint32), C.POINTER(C.c_int32)]
        L.incin_host_capability_docs.restype = C.c_size_t
        L.incin_host_capability_docs.argtypes = [C.c_char_p, C.c_size_t]
        I64P, I32P = C.POINTER(C.c_int64), C.POINTER(C.c_int32)
        L.incin_host_lower_attention.argtypes = [I64P, C.c_int32, I64P, C.c_int32, I64P, C.c_int32, C.c_int32, C.c_int32, I32P,
                                                 C.c_int64, C.c_int32, C.c_double, I32P, C.c_int64, C.POINTER(C.c_void_p)]
        L.incin_host_attention_spec_out_dims.argtypes = [C.c_void_p, I64P, I32P, I64P]
        L.incin_host_execute_attention.argtypes = [C.c_void_p, C.POINTER(C.c_void_p), C.c_int32, C.POINTER(C.c_void_p)]
        L.incin_host_release_attention_spec.restype = None
        L.incin_host_release_attention_spec.argtypes = [C.c_void_p]
        L.incin_host_reshape.argtypes = [C.c_void_p, I64P, C.c_int32, C.POINTER(C.c_void_p)]
        L.incin_host_is_compiled_in.argtypes = [C.c_int32]
        L.incin_host_probe.argtypes = [C.c_int32]
        L.incin_host_detect_device.argtypes = [I32P, C.c_int32, I32P, I32P]
        L.incin_host_data_ptr.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        L.incin_host_set_stream.restype = None
        L.incin_host_set_stream.argtypes = [C.c_void_p]
        L.incin_host_begin_recording.argtypes = [C.c_int32]
        L.incin_host_end_recording.argtypes = [C.POINTER(C.c_void_p)]
        L.incin_host_replay.argtypes = [C.c_void_p]
        L.incin_host_release_graph.restype = None
        L.incin_host_release_graph.argtypes = [C.c_void_p]
        L.incin_host_pool_stats.argtypes = [C.c_int32, I64P, I64P, I64P]
        L.incin_host_trim_pool.argtypes = [C.c_int32]
        _lib = L
    return _lib


def _check(code):
    if code != 0:
        raise BackendError(code, lib().incin_host_last_error().decode())


def _dims(dims):
    return (C.c_int64 * max(len(dims), 1))(*dims)


class RocmStorage:
    """Owns one handle of the C++ library."""

    def __init__(self, handle):
        self._h = C.c_void_p(handle)

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.incin_host_release(self._h)
            self._h = None

    # -- Backend::from_bytes / to_bytes ------------------------------------------------------------
    @classmethod
    def from_numpy(cls, a, dtype=F32, device=0):
        """`a` holds float values; they are stored on the device as `dtype` (round-to-nearest-even)."""
        a = np.asarray(a, order="C")          # (ascontiguousarray would turn a rank-0 array into rank 1)
        if dtype == F32:
            raw = a.astype(np.float32).tobytes()
        elif dtype == F16:
            raw = a.astype(np.float16).tobytes()
        elif dtype == BF16:
            raw = DT.f32_to_bf16_bits(a.astype(np.float32)).tobytes()
        else:
            raw = a.tobytes()
        return cls.from_bytes(raw, tuple(a.shape), dtype, device)

    @classmethod
    def from_bytes(cls, raw, dims, dtype, device=0):
        out = C.c_void_p()
        buf = C.create_string_buffer(raw, len(raw)) if raw else None
        _check(lib().incin_host_from_bytes(buf, len(raw), _dims(dims), len(dims), dtype, device, C.byref(out)))
        return cls(out.value)

    @property
    def shape(self):
        r = C.c_int32()
        lib().incin_host_rank(self._h, C.byref(r))
        d = (C.c_int64 * max(r.value, 1))()
        lib().incin_host_shape(self._h, d)
        return tuple(d[i] for i in range(r.value))

    @property
    def strides(self):
        """Element strides of the view (0 on a broadcast axis)."""
        n = len(self.shape)
        d = (C.c_int64 * max(n, 1))()
        lib().incin_host_strides(self._h, d)
        return tuple(d[i] for i in range(n))

    @property
    def data_ptr(self):
        p = C.c_void_p()
        lib().incin_host_data_ptr(self._h, C.byref(p))
        return p.value

    def is_contiguous(self):
        acc = 1
        for n, st in zip(reversed(self.shape), reversed(self.strides)):
            if n != 1 and st != acc:
                return False
            acc *= n
        return True

    @property
    def dtype(self):
        t = C.c_int32()
        lib().incin_host_dtype(self._h, C.byref(t))
        return t.value

    def to_bytes(self):
        n = C.c_int64()
        lib().incin_host_numel(self._h, C.byref(n))
        size = n.value * (4 if self.dtype == F32 else 2)
        buf = C.create_string_buffer(max(size, 1))
        _check(lib().incin_host_to_bytes(self._h, buf, size))
        return buf.raw[:size]

    def to_numpy(self):
        """Logical contents as float32."""
        raw = self.to_bytes()
        t = self.dtype
        if t == F32:
            a = np.frombuffer(raw, dtype=np.float32)
        elif t == F16:
            a = np.frombuffer(raw, dtype=np.float16).astype(np.float32)
        else:
            a = DT.bf16_bits_to_f32(np.frombuffer(raw, dtype=np.uint16))
        return a.reshape(self.shape).copy()

    # -- metadata-only views ---------------------------------------------------------------------------
    def _view(self, fn, *args):
        out = C.c_void_p()
        _check(fn(self._h, *args, C.byref(out)))
        return RocmStorage(out.value)

    def transpose(self, a, b):
        return self._view(lib().incin_host_transpose, a, b)

    def broadcast_as(self, dims):
        return self._view(lib().incin_host_broadcast_as, _dims(dims), len(dims))

    def narrow(self, dim, start, length):
        return self._view(lib().incin_host_narrow, dim, start, length)

    def reshape(self, dims):
        """Same elements under another shape; a view that is not dense is gathered into a dense copy first."""
        return self._view(lib().incin_host_reshape, _dims(dims), len(dims))

    def tag_causal(self):
        return self._view(lib().incin_host_tag_causal)

    def infer_mask_tag(self):
        """(storage, kind): the mask tagged with what its rows state - kind 1 causal, 2 key padding, 3 both - or, kind 0,
        the mask as it was.  Reads the mask on the device and waits for the answer: once per mask, where it is made."""
        kind = C.c_int32(0)
        out = C.c_void_p()
        _check(lib().incin_host_infer_mask_tag(self._h, C.byref(kind), C.byref(out)))
        return RocmStorage(out.value), int(kind.value)

    def tag_key_padding(self, lens):
        arr = (C.c_int32 * max(len(lens), 1))(*[int(x) for x in lens])
        return self._view(lib().incin_host_tag_key_padding, arr, len(lens))


def scaled_dot_product_attention(q, k, v, mask=None, scale=None):
    """TensorOps::scaled_dot_product_attention on the Rocm backend mirror."""
    out = C.c_void_p()
    _check(lib().incin_host_scaled_dot_product_attention(
        q._h, k._h, v._h, mask._h if mask is not None else None,
        0 if scale is None else 1, 0.0 if scale is None else float(scale), C.byref(out)))
    return RocmStorage(out.value)


def attention_backward(q, k, v, grad_out, mask=None, scale=None):
    """(out, dq, dk, dv): the operator and its gradients for an upstream gradient of the output's shape."""
    hs = [C.c_void_p() for _ in range(4)]
    _check(lib().incin_host_attention_backward(
        q._h, k._h, v._h, mask._h if mask is not None else None,
        0 if scale is None else 1, 0.0 if scale is None else float(scale), grad_out._h, *[C.byref(h) for h in hs]))
    return tuple(RocmStorage(h.value) for h in hs)


def set_stream(stream_ptr):
    """The stream the calling thread's operators launch on from now on (None: the device's default stream)."""
    lib().incin_host_set_stream(stream_ptr)


class Recording:
    """`with Recording(device) as rec:` records the calling thread's operators on its stream (set_stream) into a launch
    graph; afterwards `rec.replay()` runs them again.  The recording keeps the buffers its kernels use."""

    def __init__(self, device=0):
        self.device, self._g = device, None

    def __enter__(self):
        _check(lib().incin_host_begin_recording(self.device))
        return self

    def __exit__(self, et, ev, tb):
        g = C.c_void_p()
        code = lib().incin_host_end_recording(C.byref(g))
        if et is None:
            _check(code)
        self._g = g
        return False

    def replay(self):
        _check(lib().incin_host_replay(self._g))

    def release(self):
        if self._g:
            lib().incin_host_release_graph(self._g)
            self._g = None


def pool_stats(device=0):
    """(device allocations so far, buffers handed out from the pool, bytes idle in the pool)"""
    a, r, i = C.c_int64(), C.c_int64(), C.c_int64()
    lib().incin_host_pool_stats(device, C.byref(a), C.byref(r), C.byref(i))
    return a.value, r.value, i.value


def trim_pool(device=0):
    _check(lib().incin_host_trim_pool(device))


def last_launch_count():
    return lib().incin_host_last_launch_count()
