"""ctypes view of the descriptor / executor layer and device detection of the C++ host mirror
(incin_amd/host/rocm_exec.hpp)."""
import ctypes as C
from collections import namedtuple

from . import rocm_backend as RB
from . import rocm_capability as RC


class AttentionSpec:
    """A validated attention descriptor (`lower` is the shape rule and needs no device)."""

    def __init__(self, handle):
        self._h = handle

    def __del__(self):
        if getattr(self, "_h", None):
            RB.lib().incin_host_release_attention_spec(self._h)
            self._h = None

    @classmethod
    def lower(cls, q_dims, k_dims, v_dims, dtype=RB.F32, causal=False, kv_lens=None, scale=None, q_lens=None):
        out = C.c_void_p()
        lens = None if kv_lens is None else (C.c_int32 * max(len(kv_lens), 1))(*[int(x) for x in kv_lens])
        qlens = None if q_lens is None else (C.c_int32 * max(len(q_lens), 1))(*[int(x) for x in q_lens])
        RB._check(RB.lib().incin_host_lower_attention(
            RB._dims(q_dims), len(q_dims), RB._dims(k_dims), len(k_dims), RB._dims(v_dims), len(v_dims), dtype,
            1 if causal else 0, lens, -1 if kv_lens is None else len(kv_lens),
            0 if scale is None else 1, 0.0 if scale is None else float(scale), qlens,
            -1 if q_lens is None else len(q_lens), C.byref(out)))
        return cls(out.value)

    def _out(self):
        d = (C.c_int64 * 16)()
        r, g = C.c_int32(), C.c_int64()
        RB.lib().incin_host_attention_spec_out_dims(self._h, d, C.byref(r), C.byref(g))
        return tuple(d[i] for i in range(r.value)), g.value

    @property
    def out_dims(self):
        return self._out()[0]

    @property
    def group(self):
        return self._out()[1]

    def execute(self, *inputs):
        arr = (C.c_void_p * max(len(inputs), 1))(*[s._h for s in inputs])
        out = C.c_void_p()
        RB._check(RB.lib().incin_host_execute_attention(self._h, arr, len(inputs), C.byref(out)))
        return RB.RocmStorage(out.value)


def reshape(storage, dims):
    out = C.c_void_p()
    RB._check(RB.lib().incin_host_reshape(storage._h, RB._dims(dims), len(dims), C.byref(out)))
    return RB.RocmStorage(out.value)


def is_compiled_in(kind):
    return bool(RB.lib().incin_host_is_compiled_in(RC.devices().index(kind)))


def probe(kind):
    """Device ordinal of a usable device of that kind, or None."""
    o = RB.lib().incin_host_probe(RC.devices().index(kind))
    return None if o < 0 else o


def detect_device(preference=None):
    """(kind, ordinal) of the first kind in the preference order that probes; the CPU ends the chain."""
    k, o = C.c_int32(), C.c_int32()
    if preference is None:
        RB.lib().incin_host_detect_device(None, -1, C.byref(k), C.byref(o))
    else:
        arr = (C.c_int32 * max(len(preference), 1))(*[RC.devices().index(x) for x in preference])
        RB.lib().incin_host_detect_device(arr, len(preference), C.byref(k), C.byref(o))
    return RC.devices()[k.value], o.value
