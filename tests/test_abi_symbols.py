"""The shared libraries load without a GPU and export every entry point the
headers under include/ declare (no compute call is made here)."""
import ctypes
import os
import re

from conftest import capi, entry

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared(header, prefix):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = set(re.findall(r"\b(%s[a-z0-9_]+)\s*\(" % prefix, text))
    # function-pointer members of the api table are not symbols
    return {n for n in names if not n.endswith("_api") or n == prefix + "get_api"}


def test_array_library_exports_its_header():
    assert os.path.exists(capi.GPU_LIB), "run __graft_entry__.build() first"
    dll = ctypes.CDLL(capi.GPU_LIB)
    names = declared("hordead_gpu.h", "hgpu_")
    assert len(names) >= 50
    missing = [n for n in sorted(names) if not hasattr(dll, n)]
    assert not missing, missing


def test_host_library_exports_its_header():
    assert os.path.exists(capi.HOST_LIB), "run __graft_entry__.build() first"
    dll = ctypes.CDLL(capi.HOST_LIB)
    names = declared("hordead_host.h", "hh_")
    assert len(names) >= 50
    missing = [n for n in sorted(names) if not hasattr(dll, n)]
    assert not missing, missing


def test_api_table_is_complete():
    """Every member of the gfx950 library's function table is filled in."""
    dll = ctypes.CDLL(capi.GPU_LIB)
    dll.hgpu_get_api.restype = ctypes.c_void_p
    table = dll.hgpu_get_api()
    size = ctypes.c_size_t.from_address(table).value
    n = size // ctypes.sizeof(ctypes.c_void_p)
    slots = (ctypes.c_void_p * n).from_address(table)
    assert n >= 45 and all(slots[i] for i in range(1, n))


def test_checker_exports_the_same_abi():
    dll = ctypes.CDLL(entry.ORACLE_LIB)
    for name in ("init", "upload", "download", "contract", "gather", "scatter_add", "scatter_affine", "fused_map", "get_api"):
        assert hasattr(dll, "horc_" + name), name
