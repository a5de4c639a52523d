"""The C-ABI libraries load and export every symbol the headers under include/ declare (no GPU needed)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(header="glide_hip.h", prefix="glide_hip_"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(%s\w+)\s*\(" % prefix, text)))


def test_header_symbols_are_exported():
    from glide_amd import capi
    assert os.path.exists(capi.LIB_PATH), "build the library first (python -c 'import __graft_entry__ as g; g.build()')"
    lib = ctypes.CDLL(capi.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 20
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_every_header_has_its_library():
    """include/ holds the product boundary and the measurement yardsticks, nothing else; each is exported by its own library."""
    assert sorted(os.listdir(os.path.join(ROOT, "include"))) == ["glide_hip.h", "glide_hip_probes.h"]
    names = declared_symbols("glide_hip_probes.h", "glide_probe_")
    assert names == ["glide_probe_atomic", "glide_probe_copy_bytes", "glide_probe_gather", "glide_probe_valu"]
    path = os.path.join(ROOT, "glide_amd", "libglide_probes.so")
    assert os.path.exists(path), "build the libraries first (make -C glide_amd/csrc)"
    probes = ctypes.CDLL(path)
    assert not [n for n in names if not hasattr(probes, n)]
    # the yardsticks stay out of the product library
    from glide_amd import capi
    product = ctypes.CDLL(capi.LIB_PATH)
    assert not [n for n in names if hasattr(product, n)]
    assert not [n for n in declared_symbols() if "probe" in n]


def test_version_and_error_strings():
    from glide_amd import capi
    assert "gfx950" in capi.version()
    assert capi.error_string(0) == "success"
    assert "supported" in capi.error_string(-1)
    assert capi.error_string(-2) == "bad argument"
