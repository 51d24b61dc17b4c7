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
    lib.moba_version.restype = ctypes.c_int
    assert lib.moba_version() >= 100
    lib.moba_strerror.restype = ctypes.c_char_p
    assert lib.moba_strerror(0) == b"ok"
    assert b"argument" in lib.moba_strerror(-1)
