"""CPU-side checks of the C++ host mirror: the library loads and exports the flat C view of the
backend interface.  Nothing here touches a device."""
import os
import re

from incin_amd import rocm_backend as RB

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "incin_amd", "host", "rocm_backend_c.h")


def test_host_library_exports_every_declared_symbol():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    names = sorted(set(re.findall(r"\b(incin_host_[a-z0-9_]+)\s*\(", text)))
    L = RB.lib()
    for n in names:
        assert hasattr(L, n), "missing export %s" % n
    assert set(names) == set(RB.EXPORTS)


def test_error_kinds_follow_the_reference_variants():
    # the names of incin_core::Error's variants this path can produce (incin-core/src/err.rs:109-223)
    assert RB.KINDS[2] == "ShapeMismatch" and RB.KINDS[3] == "DTypeStorageMismatch" and RB.KINDS[4] == "DeviceMismatch"
    assert RB.KINDS[8] == "UnsupportedBackendOperation"
