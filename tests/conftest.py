import ctypes
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle_c():
    """The C restatement of the reference's native operators (oracle/hades_oracle.c), built on
    demand with the Makefile beside it."""
    odir = os.path.join(ROOT, "oracle")
    so = os.path.join(odir, "libhades_oracle.so")
    src = os.path.join(odir, "hades_oracle.c")
    if not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(src):
        subprocess.run(["make", "-C", odir], check=True, capture_output=True)
    return ctypes.CDLL(so)


class SACacheRef:
    """The reference's own cache_line class behind the sequential loops of SACacheIndex
    (oracle/ref_sacache_driver.cpp, built into oracle/_ref/ where the reference tree is present).
    Same method names as the oracle's SACacheIndexModel."""

    def __init__(self, lib, cache_size):
        import numpy as np
        self._np = np
        self._lib = lib
        self._h = ctypes.c_void_p(lib.ref_sacache_new(ctypes.c_int64(cache_size)))
        self.lines = int(lib.ref_sacache_lines(self._h))

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.ref_sacache_free(self._h)
            self._h = None

    def _in(self, ids):
        ids = self._np.ascontiguousarray(ids, dtype=self._np.int64)
        return ids, ids.ctypes.data_as(ctypes.c_void_p)

    def _batch(self, fn, ids):
        ids, p = self._in(ids)
        locs = self._np.full(ids.shape, -1, dtype=self._np.int64)
        fn(self._h, p, ctypes.c_int64(ids.size), locs.ctypes.data_as(ctypes.c_void_p))
        return locs

    def add(self, ids):
        return self._batch(self._lib.ref_sacache_add, ids)

    def lookup(self, ids):
        return self._batch(self._lib.ref_sacache_lookup, ids)

    def cudalookup(self, ids):
        return self._batch(self._lib.ref_sacache_lookup_stateless, ids)

    def reset(self, ids):
        ids, p = self._in(ids)
        self._lib.ref_sacache_reset(self._h, p, ctypes.c_int64(ids.size))

    def get_valid_entries_num(self):
        return int(self._lib.ref_sacache_valid(self._h))

    def getall(self, length):
        ids = self._np.zeros(length, dtype=self._np.int64)
        locs = self._np.full(length, -1, dtype=self._np.int64)
        k = int(self._lib.ref_sacache_getall(self._h, ids.ctypes.data_as(ctypes.c_void_p),
                                             locs.ctypes.data_as(ctypes.c_void_p),
                                             ctypes.c_int64(length)))
        return ids[:k], locs[:k]


@pytest.fixture(scope="session")
def sacache_ref():
    """Factory of SACacheRef objects; skips where oracle/_ref/libsacache_ref.so has not been
    built (it needs the reference tree at build time, not at run time)."""
    so = os.path.join(ROOT, "oracle", "_ref", "libsacache_ref.so")
    if not os.path.exists(so):
        pytest.skip("oracle/_ref/libsacache_ref.so not built (make -C oracle ref)")
    lib = ctypes.CDLL(so)
    lib.ref_sacache_new.restype = ctypes.c_void_p
    lib.ref_sacache_lines.restype = ctypes.c_int64
    lib.ref_sacache_valid.restype = ctypes.c_int64
    lib.ref_sacache_getall.restype = ctypes.c_int64
    for name in ("ref_sacache_free", "ref_sacache_add", "ref_sacache_lookup",
                 "ref_sacache_lookup_stateless", "ref_sacache_reset"):
        getattr(lib, name).restype = None
    return lambda cache_size: SACacheRef(lib, cache_size)


@pytest.fixture(scope="session")
def cuda_device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def _release_cached_memory(request):
    """After every GPU test: hand torch's cached page-locked host blocks and device blocks back.
    The host allocator never releases by itself, and the sum of page-locked memory that one
    process may hold is limited on the GPU boxes (a later pin_memory allocation is then refused)."""
    yield
    if request.node.get_closest_marker("gpu") is None:
        return
    import gc
    import torch
    if torch.cuda.is_available():
        gc.collect()
        torch.cuda.synchronize()
        if hasattr(torch._C, "_host_emptyCache"):
            torch._C._host_emptyCache()
        torch.cuda.empty_cache()
