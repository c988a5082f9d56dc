"""Set-associative index cache on the device.

`IndexCache` keeps the method names of the class the reference binds as EmbCacheLib.IndexCache
(src/pybind.cc:17-36 over SACacheIndex, src/cache/cache.h) and `LocalCache` those of its Python
wrapper (python/EmbCache/cache.py:6-31).  The reference holds the structure in host shared memory,
takes and returns CPU tensors for add / lookup / reset / getall and device tensors only for
cudalookup; here the structure lives in HBM and the fast path is device tensors in, device
tensors out, so that the lookup of a batch needs no round trip through the host
(python/EmbCache/dist_emb.py:183-185).  For unmodified reference code, add / lookup / reset /
cudalookup also accept a CPU int64 tensor: it is copied to the device and the locs come back as a
CPU tensor (the reference's `lookup(ids.cpu()).cuda()` keeps working, at the price of the copies
the reference pays too).  getall returns device tensors.

Batches are handled in input order line by line: the result of the reference with one OpenMP
thread.  Ids must be int64; negative ids are never cached (loc -1).
"""
import torch

from . import _lib
from .ops import Workspace, _i64, _opt
from .EmbCacheLib import _check, _ptr, _stream

LINE_SIZE = 8          # CACHE_LINE_SIZE, src/cache/cache_line.h:5
_LINE_BYTES = 8 * LINE_SIZE + 4 * LINE_SIZE   # sizeof(cache_line<int64, int64, 8>)


class IndexCache:
    def __init__(self, cache_size, name=None, create=True, pin_memory=False, device="cuda"):
        """cache_size entries rounded up to whole lines (cache.h:139).  `name`, `create` and
        `pin_memory` are the reference's shared-memory arguments (cache.h:145-167) and are
        accepted for signature compatibility only: the structure is private device memory."""
        _check(cache_size >= 1, "cache_size must be >= 1")
        self.device = torch.device(device)
        self.lines = (int(cache_size) + LINE_SIZE - 1) // LINE_SIZE
        self.line_ids = torch.empty(self.lines * LINE_SIZE, dtype=torch.int64, device=self.device)
        self.line_age = torch.empty(self.lines * LINE_SIZE, dtype=torch.int32, device=self.device)
        self._ws = Workspace(self.device)
        _lib.call("hades_sacache_init", _ptr(self.line_ids), _ptr(self.line_age), self.lines,
                  _stream())

    # ---- sizes (cache.h:178-194) ----
    def get_size(self):
        return self.lines * LINE_SIZE

    def get_capacity(self):
        return self.lines * LINE_SIZE

    def get_space(self):
        return self.lines * _LINE_BYTES

    def get_valid_entries_num(self):
        """Number of live entries (one host synchronisation)."""
        num_valid = torch.empty(1, dtype=torch.int64, device=self.device)
        ws = self._ws.get(_lib.query("hades_sacache_getall_workspace_bytes", self.lines))
        _lib.call("hades_sacache_getall", _ptr(self.line_ids), self.lines, None, None, None,
                  _ptr(num_valid), 0, _ptr(ws), ws.numel(), _stream())
        return int(num_valid.item())

    # ---- operations ----
    def _in(self, ids):
        """(ids on the device, whether the caller's tensor lives on the host)"""
        _check(ids.dtype == torch.int64, "ids must be int64")
        if ids.is_cuda:
            return ids, False
        return ids.contiguous().to(self.device), True

    def _ordered(self, entry, ids):
        ids, from_host = self._in(ids)
        locs = self._ordered_dev(entry, ids)
        return locs.cpu() if from_host else locs

    def _ordered_dev(self, entry, ids):
        _i64(ids, "ids")
        locs = torch.empty_like(ids)
        n = ids.numel()
        ws = self._ws.get(_lib.query("hades_sacache_workspace_bytes", n))
        _lib.call(entry, _ptr(self.line_ids), _ptr(self.line_age), self.lines, _ptr(ids), n,
                  _ptr(locs), _ptr(ws), ws.numel(), _stream())
        return locs

    def add(self, ids):
        """Inserts the ids that are absent; returns the loc of every id, -1 where its line had no
        entry to give (cache.h:51-91)."""
        return self._ordered("hades_sacache_add", ids)

    def lookup(self, ids):
        """loc or -1 per id; every hit ages its line, as the reference's host lookup does
        (cache.h:93-107)."""
        return self._ordered("hades_sacache_lookup_touch", ids)

    def cudalookup(self, ids):
        """loc or -1 per id; the cache is left as it is (src/cache/lookup.cu:15-45)."""
        ids, from_host = self._in(ids)
        _i64(ids, "ids")
        locs = torch.empty_like(ids)
        _lib.call("hades_sacache_lookup", _ptr(self.line_ids), self.lines, _ptr(ids), ids.numel(),
                  _ptr(locs), _stream())
        return locs.cpu() if from_host else locs

    def reset(self, ids):
        """Frees the entries of the ids that are present (cache.h:109-121)."""
        ids, _ = self._in(ids)
        _i64(ids, "ids")
        _lib.call("hades_sacache_reset", _ptr(self.line_ids), _ptr(self.line_age), self.lines,
                  _ptr(ids), ids.numel(), _stream())

    def getall_padded(self, length):
        """(ids int64[length], locs int64[length], num int64[1]) on the device: the first num[0]
        pairs are the live entries in loc order; no host synchronisation."""
        length = int(length)
        ids = torch.zeros(length, dtype=torch.int64, device=self.device)
        locs = torch.full((length,), -1, dtype=torch.int64, device=self.device)
        num = torch.empty(1, dtype=torch.int64, device=self.device)
        ws = self._ws.get(_lib.query("hades_sacache_getall_workspace_bytes", self.lines))
        _lib.call("hades_sacache_getall", _ptr(self.line_ids), self.lines, _opt(ids), _opt(locs),
                  _ptr(num), None, length, _ptr(ws), ws.numel(), _stream())
        return ids, locs, num

    def getall(self, length):
        """(ids, locs) of `length` elements as the reference returns them (cache.h:243-257): live
        entries first, the rest left at id 0 / loc -1."""
        ids, locs, _ = self.getall_padded(length)
        return ids, locs


class LocalCache:
    """python/EmbCache/cache.py:6-31, same methods, over the device-resident IndexCache."""

    def __init__(self, name, cache_size, create=True, pin_memory=False, device="cuda"):
        self._cache_size = cache_size
        self._idx_cache = IndexCache(cache_size, name, create, pin_memory, device=device)

    def lookup(self, ids):
        return self._idx_cache.lookup(ids)

    def cudalookup(self, ids):
        return self._idx_cache.cudalookup(ids)

    def add(self, ids):
        return self._idx_cache.add(ids)

    def get_num_entries(self):
        return self._idx_cache.get_size()

    def reset(self, ids):
        self._idx_cache.reset(ids)
