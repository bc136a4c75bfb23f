"""ctypes view of the capability registry of the C++ host mirror (incin_amd/host/rocm_capability.hpp), shaped
like the reference's API: `support(device, CapabilityQuery) -> SupportLevel`, `registrations(device)`
(crates/incin-backends/src/capability.rs:339-352, incin-core/src/exec/capability.rs:9-17,119-137)."""
import ctypes as C
from collections import namedtuple

from . import rocm_backend as RB

_OPERATION, _DTYPE, _LAYOUT, _MATH, _IMPL, _DEVICE = range(6)
_COUNTS = {_OPERATION: 24, _DTYPE: 8, _LAYOUT: 7, _MATH: 2, _IMPL: 3, _DEVICE: 5}


def _names(what):
    L = RB.lib()
    return [L.incin_host_capability_name(what, i).decode() for i in range(_COUNTS[what])]


def operations():
    return _names(_OPERATION)


def dtypes():
    return _names(_DTYPE)


def layouts():
    return _names(_LAYOUT)


def math_modes():
    return _names(_MATH)


def implementations():
    return _names(_IMPL)


def devices():
    return _names(_DEVICE)


def max_rank():
    return RB.lib().incin_host_capability_max_rank()


CapabilityQuery = namedtuple("CapabilityQuery", "operation dtype layout rank training math_mode",
                             defaults=(False, "precise"))
CapabilityRule = namedtuple("CapabilityRule", "operation dtypes layouts min_rank max_rank training math_modes implementation")
REASONS = ["Operation", "DType", "Layout", "Rank", "Training", "MathMode", "MissingDeviceFeature"]


class SupportLevel(namedtuple("SupportLevel", "level reason message")):
    """level: 'native' | 'composed' | 'fallback' | 'unsupported'; reason: the UnsupportedReason variant or None."""

    @property
    def is_supported(self):
        return self.level != "unsupported"

    @property
    def is_device_local(self):
        return self.level in ("native", "composed")


def support(device, query):
    L = RB.lib()
    why = C.c_int32(-1)
    buf = C.create_string_buffer(256)
    lv = L.incin_host_capability_support(devices().index(device), operations().index(query.operation),
                                         dtypes().index(query.dtype), layouts().index(query.layout), int(query.rank),
                                         1 if query.training else 0, math_modes().index(query.math_mode),
                                         C.byref(why), buf, len(buf))
    if lv == 3:
        return SupportLevel("unsupported", REASONS[why.value], buf.value.decode())
    return SupportLevel(implementations()[lv], None, "")


def registrations(device):
    L = RB.lib()
    dev = devices().index(device)
    out = []
    for i in range(L.incin_host_capability_rule_count(dev)):
        op, lo, hi, tr, impl = C.c_int32(), C.c_int32(), C.c_int32(), C.c_int32(), C.c_int32()
        dm, lm, mm = C.c_uint32(), C.c_uint32(), C.c_uint32()
        RB._check(L.incin_host_capability_rule(dev, i, C.byref(op), C.byref(dm), C.byref(lm), C.byref(lo), C.byref(hi),
                                               C.byref(tr), C.byref(mm), C.byref(impl)))
        pick = lambda names, mask: tuple(n for j, n in enumerate(names) if mask >> j & 1)
        out.append(CapabilityRule(operations()[op.value], pick(dtypes(), dm.value), pick(layouts(), lm.value), lo.value,
                                  hi.value, bool(tr.value), pick(math_modes(), mm.value), implementations()[impl.value]))
    return out


def docs():
    """The generated tables for what this backend adds, in the format of the reference's docs/capabilities.md."""
    L = RB.lib()
    n = L.incin_host_capability_docs(None, 0)
    buf = C.create_string_buffer(n + 1)
    L.incin_host_capability_docs(buf, n + 1)
    return buf.value.decode("utf-8")
