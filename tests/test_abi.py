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
    assert lib.hades_hash_clear(one, one, one, 1000, 8, 0, null) == 1               # not a power of two
    with pytest.raises(RuntimeError, match="power of two"):
        _lib.call("hades_hash_clear", one, one, one, 1000, 8, 0, null)
    assert lib.hades_hash_clear(one, one, one, 1024, 8, -2, null) == 1              # slot stride


def test_argument_errors_of_the_split_schedule_entry_points():
    """The listed / class / static entry points check their arguments before any HIP call."""
    lib = _lib.load()
    null = ctypes.c_void_p(0)
    one = ctypes.c_void_p(256)     # never dereferenced: the checks fail first
    # listed gather / scatter: dtype, stride, null pointers; an empty list is fine
    assert lib.hades_fetch_listed(one, 0, one, one, one, 10, one, 8, 7, null) == 1
    assert b"float or double" in lib.hades_last_error()
    assert lib.hades_fetch_listed(one, 4, one, one, one, 10, one, 8, _lib.F32, null) == 1     # stride < dim
    assert b"stride" in lib.hades_last_error()
    assert lib.hades_fetch_listed(one, 0, one, null, one, 10, one, 8, _lib.F32, null) == 1
    assert lib.hades_fetch_listed(null, 0, null, null, null, 0, null, 8, _lib.F32, null) == 0
    assert lib.hades_set_listed(one, one, 3, one, one, one, 10, 8, _lib.F32, null) == 1
    assert lib.hades_set_listed(null, null, 0, null, null, null, 0, 8, _lib.F32, null) == 0
    # listed / class Adagrad
    assert lib.hades_adagrad_update_listed(one, one, one, one, 10, 8, one, one, 4, null, 0.01, 1e-10, null) == 1
    assert lib.hades_adagrad_update_listed(one, one, one, null, 10, 8, one, one, 0, null, 0.01, 1e-10, null) == 1
    assert lib.hades_adagrad_update_listed(null, null, null, null, 0, 8, null, null, 0, null, 0.01, 1e-10, null) == 0
    assert lib.hades_adagrad_update_class(one, one, one, one, 2, 255, 10, 8, one, one, 0, null, null,
                                          null, 0, 0.01, 1e-10, null) == 1                     # which
    assert lib.hades_adagrad_update_class(one, one, one, one, 0, 255, 10, 8, one, one, 0, one, null,
                                          null, 0, 0.01, 1e-10, null) == 1                     # rows without positions
    assert b"go together" in lib.hades_last_error()
    assert lib.hades_adagrad_update_class(one, one, one, one, 0, 255, 10, 8, one, one, 0, null, null,
                                          null, 1, 0.01, 1e-10, null) == 1                     # mean without counts
    assert b"run_cnts" in lib.hades_last_error()
    assert lib.hades_adagrad_update_class(one, one, one, one, 0, 255, 10, 8, one, one, 0, null, null,
                                          one, 3, 0.01, 1e-10, null) == 1                      # average code
    # the summing forms look for their plan in the workspace: too small a one is refused
    assert lib.hades_adagrad_update_class_summing(one, one, 10, 1 << 20, one, one, 0, 255, 8, one, one, 0,
                                                  null, null, null, null, 0, 0.01, 1e-10, one, 16, null) == 3
    assert lib.hades_adam_update_class_summing(one, one, 10, 1 << 20, one, one, 0, 255, 8, one, one, one, one,
                                               0, null, null, null, null, 0, 0.01, 0.9, 0.999, 1e-8, one, 16,
                                               null) == 3
    assert lib.hades_adagrad_update_class_summing(null, null, 0, 1 << 20, null, null, 0, 255, 8, null, null, 0,
                                                  null, null, null, null, 0, 0.01, 1e-10, null, 0, null) == 0
    # listed gather restricted to a set
    assert lib.hades_fetch_listed_in_set(one, 4, one, one, one, 10, one, one, 5, one, 8, _lib.F32, null) == 1   # stride < dim
    assert lib.hades_fetch_listed_in_set(one, 0, one, one, one, 10, null, one, 5, one, 8, _lib.F32, null) == 1  # set is null
    assert lib.hades_fetch_listed_in_set(one, 0, one, one, one, 10, one, one, -1, one, 8, _lib.F32, null) == 1  # set_max
    assert lib.hades_fetch_listed_in_set(null, 0, null, null, null, 10, null, null, 0, null, 8, _lib.F32, null) == 0  # empty set
    assert lib.hades_fetch_listed_in_set(null, 0, null, null, null, 0, null, null, 5, null, 8, _lib.F32, null) == 0   # empty list
    # listed / class Adam
    assert lib.hades_adam_update_listed(one, one, one, one, 10, 8, one, one, one, one, 4, 0.01, 0.9, 0.999,
                                        1e-8, null) == 1                                       # stride < dim
    assert lib.hades_adam_update_listed(one, one, one, one, 10, 8, one, null, one, one, 0, 0.01, 0.9, 0.999,
                                        1e-8, null) == 1                                       # step table
    assert lib.hades_adam_update_listed(null, null, null, null, 0, 8, null, null, null, null, 0, 0.01, 0.9,
                                        0.999, 1e-8, null) == 0
    assert lib.hades_adam_update_class(one, one, one, one, 3, 255, 10, 8, one, one, one, one, 0, null, null,
                                       null, 0, 0.01, 0.9, 0.999, 1e-8, null) == 1             # which
    assert lib.hades_adam_update_class(one, one, one, one, 1, 255, 10, 8, one, one, one, one, 0, null, one,
                                       null, 0, 0.01, 0.9, 0.999, 1e-8, null) == 1
    assert b"go together" in lib.hades_last_error()
    assert lib.hades_adam_update_class(null, null, null, null, 0, 255, 0, 8, null, null, null, null, 0, null,
                                       null, null, 0, 0.01, 0.9, 0.999, 1e-8, null) == 0
    # lookup + split: key bits must leave room for the slots
    assert lib.hades_lookup_split(one, null, 10, one, 1 << 20, null, one, null, one, one, one, one, 8,
                                  one, 1 << 20, null) == 1
    assert b"key_bits" in lib.hades_last_error()
    assert lib.hades_lookup_split(one, null, 10, one, 100, null, one, null, one, one, one, null, 0,
                                  one, 16, null) == 3                                          # workspace
    assert lib.hades_lookup_split(one, one, 10, one, 100, null, one, null, one, one, one, one, 20,
                                  one, 1 << 20, null) == 1                  # a live count and sort keys
    assert b"cannot be combined" in lib.hades_last_error()
    # host-link grid widths: set, read back, restore the default
    assert lib.hades_set_host_link_blocks(3, 8) == 1 and lib.hades_set_host_link_blocks(0, -1) == 1
    d = _lib.query("hades_get_host_link_blocks", 0)
    assert lib.hades_set_host_link_blocks(0, 48) == 0 and _lib.query("hades_get_host_link_blocks", 0) == 48
    assert lib.hades_set_host_link_blocks(0, 0) == 0 and _lib.query("hades_get_host_link_blocks", 0) == d
    # classed combine
    assert lib.hades_combine_plan_classed(one, 10, 8, 1 << 20, 1 << 19, one, one, null, null, one, 1 << 20, null) == 1
    assert lib.hades_combine_plan_classed(one, 10, 8, 1 << 20, 1 << 21, one, one, one, null, one, 1 << 20, null) == 1
    assert lib.hades_combine_apply_class(one, 10, 8, 1 << 20, 0, 2, one, one, one, one, one, 1 << 20, null) == 1
    # static combine: refused beyond its scratch, before anything else
    assert lib.hades_combine_static(one, one, 1_000_000, 128, 0, 0, one, one, one, one, null, null) == 1
    assert b"scratch" in lib.hades_last_error()
    # pinned allocation: flags and null out pointer
    p = ctypes.c_void_p()
    assert lib.hades_host_alloc_flags(ctypes.byref(p), 16, 4) == 1
    assert lib.hades_host_alloc_flags(None, 16, 0) == 1
    assert lib.hades_host_alloc_flags(ctypes.byref(p), 0, 0) == 0 and not p.value


def test_workspace_queries():
    assert _lib.query("hades_combine_workspace_bytes", 0, 8) > 0
    a = _lib.query("hades_combine_workspace_bytes", 200_000, 128)
    b = _lib.query("hades_combine_workspace_bytes", 1_000_000, 128)
    assert 0 < a < b
    assert _lib.query("hades_split_compact_workspace_bytes", 1_000_000) >= 1_000_000
    assert _lib.query("hades_hash_flush_workspace_bytes", 1 << 22, 1 << 22) > (1 << 22) * 8


def test_interface_version_agrees_between_header_binding_and_library():
    """HADES_ABI_VERSION of the header, the number the Python binding expects and what the built
    library reports are one number: a library built from other sources is refused at load."""
    import re
    from hades_amd import _lib
    header = open(os.path.join(ROOT, "include", "hades_hip.h")).read()
    v = int(re.search(r"#define HADES_ABI_VERSION (\d+)", header).group(1))
    assert v == _lib.ABI_VERSION == _lib.load().hades_version()
