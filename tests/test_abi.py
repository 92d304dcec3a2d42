"""The C-ABI library loads without a GPU and exports every symbol the header declares."""
import ctypes
import os
import re

import pytest

from aici_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "hipattn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hipattn_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    lib = _lib.load()
    declared = _declared_symbols()
    assert len(declared) >= 50
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in hipattn.h but not exported"
    # the Python binding covers exactly the header
    assert sorted(_lib.EXPORTED_SYMBOLS) == declared


def test_version_and_error_convention_on_host_only_calls():
    lib = _lib.load()
    assert lib.hipattn_version().decode() == "0.1.0"
    h = ctypes.c_void_p()
    with pytest.raises(_lib.HipAttnError, match="bad geometry"):
        _lib.call("hipattn_block_allocator_new", 0, 4, ctypes.byref(h))
    # argument validation happens before any GPU work, so it is testable here
    t = _lib.Tensor()
    t.ndim = 2
    with pytest.raises(_lib.HipAttnError, match="expected 3 dims"):
        _lib.call("hipattn_mha_varlen_fwd", ctypes.pointer(t), None, None, None, None, None, 1, 1, 0.0, 1.0, False,
                  True, -1, -1, None, None, None)
    with pytest.raises(_lib.HipAttnError, match="NULL"):
        _lib.call("hipattn_reshape_and_cache", None, None, None, None, None, None)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "libhipattn.so")
    with pytest.raises(ImportError, match="not built"):
        _lib.load()
