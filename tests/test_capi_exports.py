"""The C-ABI library loads and exports every symbol include/glide_hip.h declares (no GPU needed)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "glide_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(glide_hip_\w+)\s*\(", text)))


def test_header_symbols_are_exported():
    from glide_amd import capi
    assert os.path.exists(capi.LIB_PATH), "build the library first (python -c 'import __graft_entry__ as g; g.build()')"
    lib = ctypes.CDLL(capi.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 20
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_version_and_error_strings():
    from glide_amd import capi
    assert "gfx950" in capi.version()
    assert capi.error_string(0) == "success"
    assert "supported" in capi.error_string(-1)
    assert capi.error_string(-2) == "bad argument"
