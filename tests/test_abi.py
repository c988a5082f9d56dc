"""The C-ABI library loads and exports every symbol include/hades_hip.h declares; argument
checks that need no GPU return error codes and messages instead of exiting.  No GPU."""
import ctypes
import os
import re

import pytest

from hades_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "hades_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hades_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 30
    for name in names:
        assert hasattr(lib, name), "libhades_hip.so does not export %s" % name
    assert set(names) == set(_lib.exported_names())


def test_library_has_no_torch_or_oracle_dependency():
    import subprocess
    out = subprocess.run(["ldd", _lib.LIB_PATH], capture_output=True, text=True).stdout
    assert "libamdhip64" in out
    assert "torch" not in out and "oracle" not in out


def test_argument_errors_are_codes_and_messages():
    lib = _lib.load()
    null = ctypes.c_void_p(0)
    one = ctypes.c_void_p(16)      # never dereferenced: the checks fail first
    assert lib.hades_fetch2(one, one, one, 4, 8, 7, _lib.I64, null) == 1      # bad dtype code
    assert b"float or double" in lib.hades_last_error()
    assert lib.hades_fetch2(one, one, one, 4, 8, _lib.F32, 9, null) == 1      # bad index code
    assert b"int32 or int64" in lib.hades_last_error()
    assert lib.hades_fetch2(one, one, one, -1, 8, _lib.F32, _lib.I64, null) == 1
    assert lib.hades_fetch2(null, one, one, 4, 8, _lib.F32, _lib.I64, null) == 1
    assert lib.hades_fetch2(null, null, null, 0, 8, _lib.F32, _lib.I64, null) == 0   # empty batch
    assert lib.hades_combine(one, one, 1 << 30, 8, 0, 0, one, one, one, one, null, one, 1 << 20, null) == 1
    assert lib.hades_combine(one, one, 10, 8, 0, 5, one, one, one, one, null, one, 1 << 20, null) == 1
    assert lib.hades_combine(one, one, 10, 8, 0, 0, one, one, one, one, null, one, 16, null) == 3
    assert b"workspace too small" in lib.hades_last_error()
    assert lib.hades_hash_clear(one, one, one, 1000, 8, null) == 1                  # not a power of two
    with pytest.raises(RuntimeError, match="power of two"):
        _lib.call("hades_hash_clear", one, one, one, 1000, 8, null)


def test_workspace_queries():
    assert _lib.query("hades_combine_workspace_bytes", 0, 8) > 0
    a = _lib.query("hades_combine_workspace_bytes", 200_000, 128)
    b = _lib.query("hades_combine_workspace_bytes", 1_000_000, 128)
    assert 0 < a < b
    assert _lib.query("hades_split_compact_workspace_bytes", 1_000_000) >= 1_000_000
    assert _lib.query("hades_hash_flush_workspace_bytes", 1 << 22, 1 << 22) > (1 << 22) * 8
