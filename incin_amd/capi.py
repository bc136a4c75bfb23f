"""ctypes binding of the C ABI in include/incin_rocm.h.

This is the thin Python mirror of what a Rust `incin-rocm-sys` crate binds: one
function per exported symbol, the descriptor struct, and an exception that
carries the library's status code and message.  There is no fallback: if the
shared library is missing, loading raises.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# INCIN_ROCM_LIBRARY overrides the in-tree location (e.g. to load an installed or experimental build)
LIB_PATH = os.environ.get("INCIN_ROCM_LIBRARY") or os.path.join(_HERE, "lib", "libincin_rocm.so")

F32, F16, BF16 = 0, 1, 2
IMPL_AUTO, IMPL_GENERIC, IMPL_MFMA, IMPL_SPLITKV, IMPL_MFMA64, IMPL_SPLITKV_MFMA = 0, 1, 2, 3, 4, 5
OK, EINVAL, ESHAPE, EDTYPE, EDEVICE, ENOMEM, EWORKSPACE, EUNSUPPORTED, ERUNTIME = range(9)

EXPORTS = [
    "incin_rocm_last_error", "incin_rocm_abi_version",
    "incin_rocm_sizeof_sdpa_desc", "incin_rocm_sizeof_device_info",
    "incin_rocm_device_count", "incin_rocm_device_info",
    "incin_rocm_alloc", "incin_rocm_free", "incin_rocm_memset",
    "incin_rocm_memcpy_h2d", "incin_rocm_memcpy_d2h", "incin_rocm_memcpy_d2d", "incin_rocm_copy_strided", "incin_rocm_sum_to_shape", "incin_rocm_mask_row_limits", "incin_rocm_sync",
    "incin_rocm_stream_create", "incin_rocm_stream_destroy", "incin_rocm_stream_sync",
    "incin_rocm_event_create", "incin_rocm_event_destroy", "incin_rocm_event_record",
    "incin_rocm_event_sync", "incin_rocm_event_query", "incin_rocm_event_elapsed_ms",
    "incin_rocm_graph_begin", "incin_rocm_graph_end", "incin_rocm_graph_launch", "incin_rocm_graph_destroy",
    "incin_rocm_sdpa_workspace", "incin_rocm_sdpa_fwd", "incin_rocm_sdpa_fwd_static",
    "incin_rocm_sizeof_kv_append_desc", "incin_rocm_kv_append",
    "incin_rocm_sizeof_sdpa_bwd_desc", "incin_rocm_sdpa_bwd_workspace", "incin_rocm_sdpa_bwd",
    "incin_rocm_matrix_rate", "incin_rocm_read_rate", "incin_rocm_lds_fill",
]


class DeviceInfo(C.Structure):
    _fields_ = [
        ("name", C.c_char * 64),
        ("arch", C.c_char * 32),
        ("compute_units", C.c_int32),
        ("clock_khz", C.c_int32),
        ("memory_clock_khz", C.c_int32),
        ("memory_bus_bits", C.c_int32),
        ("lds_bytes_per_block", C.c_int32),
        ("wavefront_size", C.c_int32),
        ("hbm_bytes", C.c_uint64),
    ]


class SdpaDesc(C.Structure):
    _fields_ = [
        ("dtype", C.c_int32),
        ("device", C.c_int32),
        ("B", C.c_int64), ("Hq", C.c_int64), ("Hkv", C.c_int64),
        ("Sq", C.c_int64), ("Skv", C.c_int64), ("D", C.c_int64), ("Dv", C.c_int64),
        ("q_stride", C.c_int64 * 3),
        ("k_stride", C.c_int64 * 3),
        ("v_stride", C.c_int64 * 3),
        ("o_stride", C.c_int64 * 3),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p),
        ("scale", C.c_float),
        ("causal", C.c_int32),
        ("kv_lens", C.c_void_p),
        ("add_mask", C.c_void_p),
        ("mask_stride", C.c_int64 * 4),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_size_t),
        ("num_splits", C.c_int32),
        ("impl", C.c_int32),
        ("q_lens", C.c_void_p),
        ("lse", C.c_void_p),
    ]


class SdpaBwdDesc(C.Structure):
    _fields_ = [
        ("fwd", SdpaDesc),
        ("d_o", C.c_void_p), ("d_o_stride", C.c_int64 * 3),
        ("d_q", C.c_void_p), ("d_q_stride", C.c_int64 * 3),
        ("d_k", C.c_void_p), ("d_k_stride", C.c_int64 * 3),
        ("d_v", C.c_void_p), ("d_v_stride", C.c_int64 * 3),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_size_t),
    ]


class KvAppendDesc(C.Structure):
    _fields_ = [
        ("dtype", C.c_int32),
        ("device", C.c_int32),
        ("B", C.c_int64), ("Hkv", C.c_int64), ("S_new", C.c_int64), ("S_max", C.c_int64), ("D", C.c_int64), ("Dv", C.c_int64),
        ("k_new", C.c_void_p), ("v_new", C.c_void_p),
        ("k_new_stride", C.c_int64 * 3), ("v_new_stride", C.c_int64 * 3),
        ("k_cache", C.c_void_p), ("v_cache", C.c_void_p),
        ("k_cache_stride", C.c_int64 * 3), ("v_cache_stride", C.c_int64 * 3),
        ("kv_lens", C.c_void_p),
    ]


class RocmError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("incin_rocm error %d: %s" % (code, message))
        self.code = code
        self.message = message


_lib = None


def load():
    """Load libincin_rocm.so; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "libincin_rocm.so is not built (%s); run `python -m incin_amd.build`. "
            "There is no CPU fallback for this backend." % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    lib.incin_rocm_last_error.restype = C.c_char_p
    for name in EXPORTS[1:]:
        getattr(lib, name).restype = C.c_int
    lib.incin_rocm_sizeof_sdpa_desc.restype = C.c_size_t
    lib.incin_rocm_sizeof_device_info.restype = C.c_size_t
    if lib.incin_rocm_sizeof_sdpa_desc() != C.sizeof(SdpaDesc) or lib.incin_rocm_sizeof_device_info() != C.sizeof(DeviceInfo):
        raise RuntimeError("libincin_rocm.so was built from a different include/incin_rocm.h than this binding mirrors")
    lib.incin_rocm_alloc.argtypes = [C.c_int32, C.c_size_t, C.POINTER(C.c_void_p)]
    lib.incin_rocm_free.argtypes = [C.c_int32, C.c_void_p]
    lib.incin_rocm_memset.argtypes = [C.c_int32, C.c_void_p, C.c_int, C.c_size_t]
    for name in ("incin_rocm_memcpy_h2d", "incin_rocm_memcpy_d2h", "incin_rocm_memcpy_d2d"):
        getattr(lib, name).argtypes = [C.c_int32, C.c_void_p, C.c_void_p, C.c_size_t]
    lib.incin_rocm_sync.argtypes = [C.c_int32]
    lib.incin_rocm_copy_strided.argtypes = [C.c_int32, C.c_void_p, C.c_void_p, C.c_int32, C.POINTER(C.c_int64), C.POINTER(C.c_int64),
                                            C.c_int32, C.c_void_p]
    lib.incin_rocm_mask_row_limits.argtypes = [C.c_int32, C.c_int32, C.c_void_p, C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.c_void_p, C.c_void_p]
    lib.incin_rocm_sum_to_shape.argtypes = [C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_int32, C.POINTER(C.c_int64), C.POINTER(C.c_int64),
                                            C.c_void_p]
    lib.incin_rocm_device_count.argtypes = [C.POINTER(C.c_int32)]
    lib.incin_rocm_device_info.argtypes = [C.c_int32, C.POINTER(DeviceInfo)]
    lib.incin_rocm_stream_create.argtypes = [C.c_int32, C.POINTER(C.c_void_p)]
    lib.incin_rocm_stream_destroy.argtypes = [C.c_int32, C.c_void_p]
    lib.incin_rocm_stream_sync.argtypes = [C.c_int32, C.c_void_p]
    lib.incin_rocm_event_create.argtypes = [C.c_int32, C.POINTER(C.c_void_p)]
    lib.incin_rocm_event_destroy.argtypes = [C.c_int32, C.c_void_p]
    lib.incin_rocm_event_record.argtypes = [C.c_int32, C.c_void_p, C.c_void_p]
    lib.incin_rocm_event_sync.argtypes = [C.c_int32, C.c_void_p]
    lib.incin_rocm_event_query.argtypes = [C.c_int32, C.c_void_p, C.POINTER(C.c_int32)]
    lib.incin_rocm_event_elapsed_ms.argtypes = [C.c_int32, C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]
    lib.incin_rocm_graph_begin.argtypes = [C.c_int32, C.c_void_p]
    lib.incin_rocm_graph_end.argtypes = [C.c_int32, C.c_void_p, C.POINTER(C.c_void_p)]
    lib.incin_rocm_graph_launch.argtypes = [C.c_int32, C.c_void_p, C.c_void_p]
    lib.incin_rocm_graph_destroy.argtypes = [C.c_int32, C.c_void_p]
    lib.incin_rocm_sdpa_workspace.argtypes = [C.POINTER(SdpaDesc), C.POINTER(C.c_size_t), C.POINTER(C.c_int32),
                                              C.POINTER(C.c_int32)]
    lib.incin_rocm_sdpa_fwd.argtypes = [C.POINTER(SdpaDesc), C.c_void_p]
    lib.incin_rocm_sdpa_fwd_static.argtypes = [C.POINTER(SdpaDesc), C.c_void_p]
    lib.incin_rocm_sizeof_kv_append_desc.restype = C.c_size_t
    lib.incin_rocm_sizeof_sdpa_bwd_desc.restype = C.c_size_t
    lib.incin_rocm_sdpa_bwd_workspace.argtypes = [C.POINTER(SdpaBwdDesc), C.POINTER(C.c_size_t)]
    lib.incin_rocm_sdpa_bwd.argtypes = [C.POINTER(SdpaBwdDesc), C.c_void_p]
    lib.incin_rocm_kv_append.argtypes = [C.POINTER(KvAppendDesc), C.c_void_p]
    lib.incin_rocm_matrix_rate.argtypes = [C.c_int32, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.POINTER(C.c_double), C.c_void_p]
    lib.incin_rocm_read_rate.argtypes = [C.c_int32, C.c_void_p, C.c_size_t, C.c_int32, C.c_void_p, C.c_void_p]
    lib.incin_rocm_lds_fill.argtypes = [C.c_int32, C.c_uint32, C.c_void_p, C.c_void_p]
    _lib = lib
    return lib


def check(rc):
    if rc != 0:
        raise RocmError(rc, load().incin_rocm_last_error().decode("utf-8", "replace"))


def device_count():
    n = C.c_int32(0)
    check(load().incin_rocm_device_count(C.byref(n)))
    return n.value


def device_info(dev=0):
    info = DeviceInfo()
    check(load().incin_rocm_device_info(dev, C.byref(info)))
    return info


class DeviceBuffer:
    """Owns one device allocation (the role of CudaBuffer in cuda/storage.rs:24-59)."""

    def __init__(self, nbytes, dev=0):
        self.dev = dev
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(load().incin_rocm_alloc(dev, self.nbytes, C.byref(p)))
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, arr, dev=0):
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes, dev)
        if arr.nbytes:
            check(load().incin_rocm_memcpy_h2d(dev, buf.ptr, arr.ctypes.data, arr.nbytes))
        return buf

    def to_numpy(self, dtype, shape):
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        if out.nbytes:
            check(load().incin_rocm_memcpy_d2h(self.dev, out.ctypes.data, self.ptr, out.nbytes))
        return out

    def free(self):
        if self.ptr:
            check(load().incin_rocm_free(self.dev, self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def sync(dev=0):
    check(load().incin_rocm_sync(dev))


def sdpa_workspace(desc):
    nbytes, splits, impl = C.c_size_t(0), C.c_int32(0), C.c_int32(0)
    check(load().incin_rocm_sdpa_workspace(C.byref(desc), C.byref(nbytes), C.byref(splits), C.byref(impl)))
    return nbytes.value, splits.value, impl.value


def sdpa_bwd_workspace(desc):
    n = C.c_size_t()
    check(load().incin_rocm_sdpa_bwd_workspace(C.byref(desc), C.byref(n)))
    return n.value


def sdpa_bwd(desc, stream=None):
    check(load().incin_rocm_sdpa_bwd(C.byref(desc), stream))


def read_rate(src, nbytes, nontemporal, sink, stream=None, dev=0):
    """One launch of the read-only kernel over nbytes of src (DeviceBuffer); time it with events."""
    check(load().incin_rocm_read_rate(dev, src.ptr, nbytes, 1 if nontemporal else 0, sink.ptr, stream))


def lds_fill(pattern, sink, stream=None, dev=0):
    """Writes the 32-bit pattern into the whole LDS of every compute unit (sink: a DeviceBuffer of 4 bytes or more)."""
    check(load().incin_rocm_lds_fill(dev, pattern, sink.ptr, stream))


def matrix_rate(operands, sink, mix, iterations, stream=None, dev=0):
    """One launch of the matrix-instruction loop on the 256 KiB at `operands`; returns the FLOPs of the launch."""
    fl = C.c_double(0.0)
    check(load().incin_rocm_matrix_rate(dev, operands.ptr, sink.ptr, mix, iterations, C.byref(fl), stream))
    return fl.value


def kv_append(desc, stream=None):
    check(load().incin_rocm_kv_append(C.byref(desc), stream))


def sdpa_fwd(desc, stream=None):
    check(load().incin_rocm_sdpa_fwd(C.byref(desc), stream))


STATIC_SCRATCH_BYTES = 8 << 20      # INCIN_ROCM_STATIC_SCRATCH_BYTES


def sdpa_fwd_static(desc, stream=None):
    """incin_rocm_sdpa_fwd_static: the launch that takes its scratch memory from the library's static buffer."""
    check(load().incin_rocm_sdpa_fwd_static(C.byref(desc), stream))


class Event:
    def __init__(self, dev=0):
        self.dev = dev
        p = C.c_void_p()
        check(load().incin_rocm_event_create(dev, C.byref(p)))
        self.ptr = p.value

    def record(self, stream=None):
        check(load().incin_rocm_event_record(self.dev, self.ptr, stream))

    def sync(self):
        check(load().incin_rocm_event_sync(self.dev, self.ptr))

    def elapsed_ms(self, stop):
        ms = C.c_float(0)
        check(load().incin_rocm_event_elapsed_ms(self.dev, self.ptr, stop.ptr, C.byref(ms)))
        return ms.value

    def destroy(self):
        if self.ptr:
            check(load().incin_rocm_event_destroy(self.dev, self.ptr))
            self.ptr = None


class Stream:
    def __init__(self, dev=0):
        self.dev = dev
        p = C.c_void_p()
        check(load().incin_rocm_stream_create(dev, C.byref(p)))
        self.ptr = p.value

    def sync(self):
        check(load().incin_rocm_stream_sync(self.dev, self.ptr))

    def destroy(self):
        if self.ptr:
            check(load().incin_rocm_stream_destroy(self.dev, self.ptr))
            self.ptr = None


class Graph:
    """Launches recorded on a stream (`with Graph.record(stream) as g: ...`), replayed with `launch`."""

    def __init__(self, stream):
        self.dev, self.stream, self.ptr = stream.dev, stream, None

    @classmethod
    def record(cls, stream):
        return cls(stream)

    def __enter__(self):
        check(load().incin_rocm_graph_begin(self.dev, self.stream.ptr))
        return self

    def __exit__(self, exc_type, exc, tb):
        p = C.c_void_p()
        rc = load().incin_rocm_graph_end(self.dev, self.stream.ptr, C.byref(p))
        if exc_type is None:
            check(rc)
            self.ptr = p.value
        return False

    def launch(self, stream=None):
        check(load().incin_rocm_graph_launch(self.dev, self.ptr, (stream or self.stream).ptr))

    def destroy(self):
        if self.ptr:
            check(load().incin_rocm_graph_destroy(self.dev, self.ptr))
            self.ptr = None
