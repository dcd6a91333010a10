"""CPU-side checks of the C ABI: the library loads and exports every symbol that
include/smore_amd.h declares, and the ctypes table covers the same set."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "smore_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(smx_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    from smore_amd import _lib
    names = _declared()
    assert len(names) >= 7
    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail("libsmore_amd.so is not built (run __graft_entry__.build())")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == names


def test_host_only_entry_points():
    from smore_amd import _lib
    lib = _lib.load()
    assert lib.smx_version() >= 1
    assert lib.smx_kind_from_name(b"box_out") == 2
    assert lib.smx_kind_from_name(b"beta_fisher_approx") == 9
    assert lib.smx_kind_from_name(b"nope") == -1


def test_missing_library_fails_loudly(monkeypatch):
    from smore_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libsmore_amd.so")
    with pytest.raises(_lib.SmxError):
        _lib.load()
