"""The C-ABI library loads and exports every symbol declared in include/subspec_hip.h (no compute
calls, so this runs without a GPU)."""
import os

import pytest

from subspec_amd import _lib as L


def test_library_exports_every_declared_symbol():
    if not os.path.exists(L.LIB_PATH):
        import __graft_entry__ as ge
        ge.build()
    lib = L.lib()
    names = L.declared_symbols()
    assert "subspec_tree_verify" in names and "subspec_kv_compact" in names
    for name in names:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
        assert name in L._SIGNATURES, f"{name} has no ctypes signature"
    assert lib.subspec_abi_version() == 2


def test_argument_errors_are_reported_without_a_gpu():
    lib = L.lib()
    # null pointers / bad dtype are rejected on the host before any launch
    assert lib.subspec_tree_verify(None, 7, 1, 1, 1, None, None, 1, 0, 0, -1, 0, 0, 0.0, 1, 0, None, 0,
                                   None, None, None, None, None, None, None) == -1
    assert b"dtype" in lib.subspec_last_error()
    assert lib.subspec_kv_compact(None, None, 1, 0, 1, 16, 0, None, None, 0, 0, None) == -1
    with pytest.raises(ValueError):
        L.check(-1, "x")
