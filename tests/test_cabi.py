"""The C-ABI library loads and exports every symbol include/moba_hip.h declares
(no compute calls: this runs without a GPU)."""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "moba_amd", "libmoba_hip.so")
HDR = os.path.join(ROOT, "include", "moba_hip.h")


def declared_symbols():
    text = open(HDR).read()
    return sorted(set(re.findall(r"\b(moba_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        import __graft_entry__ as entry
        entry.build()
    return ctypes.CDLL(LIB)


def test_header_symbols_exported(lib):
    names = declared_symbols()
    assert len(names) >= 8
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/moba_hip.h but not exported"


def test_binding_covers_header():
    from moba_amd import _lib
    assert sorted(_lib.exported_symbols()) == declared_symbols()


def test_version_and_strerror(lib):
    from moba_amd import _lib
    lib.moba_version.restype = ctypes.c_int
    header = open(os.path.join(os.path.dirname(__file__), "..", "include", "moba_hip.h")).read()
    assert f"#define MOBA_ABI_VERSION {_lib.ABI_VERSION} " in header
    assert lib.moba_version() == _lib.ABI_VERSION
    lib.moba_strerror.restype = ctypes.c_char_p
    assert lib.moba_strerror(0) == b"ok"
    assert b"argument" in lib.moba_strerror(-1)


def _header_prototypes():
    """name -> list of parameter type strings, parsed from the header's declarations."""
    text = re.sub(r"/\*.*?\*/", " ", open(HDR).read(), flags=re.S)
    protos = {}
    for m in re.finditer(r"\b(?:int|size_t|const char\s*\*)\s*(moba_[a-z0-9_]+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        params = [p.strip() for p in m.group(2).replace("\n", " ").split(",")]
        protos[m.group(1)] = [] if params == ["void"] else params
    return protos


def test_binding_signatures_match_header():
    """Every ctypes signature has the header's number of parameters, pointer for pointer and
    integer width for integer width (a binding out of step with the header would hand the kernels
    garbage pointers)."""
    from moba_amd import _lib
    protos = _header_prototypes()
    assert sorted(protos) == declared_symbols()
    for name, (_, argtypes) in _lib._SIGNATURES.items():
        params = protos[name]
        assert len(params) == len(argtypes), (name, len(params), len(argtypes))
        for p, a in zip(params, argtypes):
            if "*" in p:
                want = (ctypes.c_void_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_int64))
            elif p.startswith("int64_t"):
                want = (ctypes.c_int64,)
            elif p.startswith("size_t"):
                want = (ctypes.c_size_t,)
            elif p.startswith("float"):
                want = (ctypes.c_float,)
            else:
                assert p.startswith("int "), (name, p)
                want = (ctypes.c_int,)
            assert a in want, (name, p, a)
