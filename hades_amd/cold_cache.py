"""The cold-data cache of the reference's cache server, resident on the device.

`ColdDataCache` holds what EmbCacheServer._create_cache allocates (python/EmbCache/server.py:
76-175) - the set-associative index, the cached embedding rows, the gradient rows with their
counts, ids, iteration counts and thresholds, and the dense buffers of the partition's own cold
rows - and offers the server's three gradient-path steps as methods:

    update_cache(ids, embs)                      server.py:499-544   (_update_cache, one client)
    accumulate_gradients_cold_remote(id, grad)   server.py:546-562
    accumulate_gradients_cold_local(id, grad)    server.py:564-574
    staled_gradients_remote() / _local()         server.py:346-419 / :421-497 (_send_staled_gradients,
                                                 without the per-client shared-memory hand-over)

The reference runs these on the CPU over shared-memory tensors, one torch indexing call at a
time, inside a server process that talks to the trainers over sockets; the process, the sockets
and the shared memory are not part of this build.  Here every step is a few kernels on the
current stream and nothing synchronises with the host except the trimmed return of the flushes.
"""
import torch

from . import _lib
from .EmbCacheLib import _check, _dev, _ptr, _stream
from .index_cache import IndexCache
from .ops import Workspace, _i64, _opt


def staleness_threshold(hotness):
    """Iterations a row may wait: ceil(1 / (0.001 + hotness)) capped at 100 (server.py:87-88)."""
    return (1 / (0.001 + hotness)).ceil().int().clamp(max=100)


class ColdDataCache:
    def __init__(self, cache_size, dim, hotness, cnt_threshold=16, part_start=0, part_nnodes=0,
                 device="cuda"):
        """cache_size: entries of the index cache (rounded up to lines of 8); hotness: float
        tensor over all ids (the per-id threshold is derived from it, server.py:87-88);
        cnt_threshold: accumulated count that forces a row out (dist_emb.py:139 passes 16);
        part_start / part_nnodes: id range of the partition's own cold rows (server.py:141-142)."""
        self.device = torch.device(device)
        self.dim = int(dim)
        self.cnt_threshold = int(cnt_threshold)
        self.threshold = staleness_threshold(hotness.to(self.device, torch.float32)).contiguous()
        self.index = IndexCache(cache_size, device=self.device)
        S = self.index.get_size()
        self.num_slots = S
        f32 = dict(dtype=torch.float32, device=self.device)
        i32 = dict(dtype=torch.int32, device=self.device)
        self.emb_cache_buff = torch.zeros((S, self.dim), **f32)          # server.py:101-105
        self.grad_cache_buff = torch.zeros((S, self.dim), **f32)         # :108-112
        self.grad_cnt_cache_buff = torch.zeros(S, **i32)                 # :115-121
        self.grad_iter_count = torch.zeros(S, **i32)                     # :124-125
        self.grad_iter_threshold = torch.zeros(S, **i32)                 # :127 (written on accumulate)
        self.grad_idx_cache_buff = torch.full((S,), -1, dtype=torch.int64, device=self.device)  # :132-139
        self.part_start, self.part_nnodes = int(part_start), int(part_nnodes)
        if self.part_nnodes:
            P = self.part_nnodes
            self.local_grad_buff = torch.zeros((P, self.dim), **f32)     # :144-149
            self.local_grad_cnt_buff = torch.zeros(P, **i32)             # :151-157
            self.local_grad_iter_count = torch.zeros(P, **i32)           # :160-161
            self.local_grad_iter_threshold = \
                self.threshold[self.part_start:self.part_start + P].contiguous()   # :164-166
        self._ws = Workspace(self.device)

    # ---- cached embedding rows -------------------------------------------------
    def update_cache(self, ids, embs):
        """Inserts the rows of one client (server.py:510-541): ids that get an entry have their
        row stored and their gradient slot cleared.  Returns the locs (-1: not cached).  ids must
        be distinct."""
        _i64(ids, "ids"); _dev(embs, "embs")
        _check(embs.dtype == torch.float32 and embs.dim() == 2 and embs.size(1) == self.dim
               and embs.size(0) == ids.numel(), "embs must be float32 [len(ids), dim]")
        locs = self.index.add(ids)
        _lib.call("hades_coldcache_insert", _ptr(locs), _ptr(ids), _ptr(self.index.line_ids),
                  _ptr(embs), ids.numel(), self.dim, self.num_slots, _ptr(self.emb_cache_buff), _ptr(self.grad_cache_buff),
                  _ptr(self.grad_cnt_cache_buff), _ptr(self.grad_idx_cache_buff), _stream())
        return locs

    def lookup(self, ids):
        """locs of the ids for the trainers' read path (python/EmbCache/client.py:116,
        dist_emb.py:183-185): -1 where the row is not cached; hits age their line."""
        return self.index.lookup(ids)

    # ---- gradient accumulation ---------------------------------------------------
    def accumulate_gradients_cold_remote(self, id, grad):
        """server.py:546-562; ids must be distinct (the reference's own assumption, :547)."""
        _i64(id, "id"); _dev(grad, "grad")
        _check(grad.dtype == torch.float32 and grad.dim() == 2 and grad.size(1) == self.dim
               and grad.size(0) == id.numel(), "grad must be float32 [len(id), dim]")
        locs = self.index.lookup(id)
        _lib.call("hades_coldcache_accumulate", _ptr(locs), _ptr(id), _ptr(grad), id.numel(),
                  self.dim, 0, self.num_slots, _ptr(self.threshold), _ptr(self.grad_cache_buff),
                  _ptr(self.grad_cnt_cache_buff), _ptr(self.grad_idx_cache_buff),
                  _ptr(self.grad_iter_threshold), _stream())
        return locs

    def accumulate_gradients_cold_local(self, id, grad):
        """server.py:564-574: the partition's own rows, addressed by id - part_start."""
        _check(self.part_nnodes > 0, "this cache was built without a local partition")
        _i64(id, "id"); _dev(grad, "grad")
        _check(grad.dtype == torch.float32 and grad.dim() == 2 and grad.size(1) == self.dim
               and grad.size(0) == id.numel(), "grad must be float32 [len(id), dim]")
        _lib.call("hades_coldcache_accumulate", None, _ptr(id), _ptr(grad), id.numel(), self.dim,
                  self.part_start, self.part_nnodes, None, _ptr(self.local_grad_buff),
                  _ptr(self.local_grad_cnt_buff), None, None, _stream())

    # ---- flush by the staleness rule ---------------------------------------------
    def _flush(self, num_slots, id_offset, buf, cnt, idx, it, thr, with_index, cap):
        cap = num_slots if cap is None else int(cap)
        out_ids = torch.empty(cap, dtype=torch.int64, device=self.device)
        out_grads = torch.empty((cap, self.dim), dtype=torch.float32, device=self.device)
        out_cnts = torch.empty(cap, dtype=torch.int64, device=self.device)
        num_out = torch.empty(1, dtype=torch.int64, device=self.device)
        ws = self._ws.get(_lib.query("hades_coldcache_flush_workspace_bytes", num_slots))
        _lib.call("hades_coldcache_flush", num_slots, self.dim, self.cnt_threshold, id_offset,
                  _ptr(buf), _ptr(cnt), _opt(idx), _ptr(it), _ptr(thr),
                  _ptr(self.index.line_ids) if with_index else None,
                  _ptr(self.index.line_age) if with_index else None,
                  self.index.lines if with_index else 0,
                  _ptr(out_ids), _ptr(out_grads), _ptr(out_cnts), _ptr(num_out), cap,
                  _ptr(ws), ws.numel(), _stream())
        return out_ids, out_grads, out_cnts, num_out

    def staled_gradients_remote_padded(self, cap=None):
        """The cached remote rows that are due (server.py:350-357), in slot order, as
        (ids[cap], grads[cap, dim], cnts[cap], num[1]) on the device; the rows are cleared and
        their ids leave the index cache (:413-419)."""
        return self._flush(self.num_slots, 0, self.grad_cache_buff, self.grad_cnt_cache_buff,
                           self.grad_idx_cache_buff, self.grad_iter_count,
                           self.grad_iter_threshold, True, cap)

    def staled_gradients_local_padded(self, cap=None):
        """The partition's own rows that are due (server.py:424-433), ids = slot + part_start."""
        _check(self.part_nnodes > 0, "this cache was built without a local partition")
        return self._flush(self.part_nnodes, self.part_start, self.local_grad_buff,
                           self.local_grad_cnt_buff, None, self.local_grad_iter_count,
                           self.local_grad_iter_threshold, False, cap)

    @staticmethod
    def _trim(out):
        ids, grads, cnts, num = out
        k = int(num.item())
        return ids[:k], grads[:k], cnts[:k]

    def staled_gradients_remote(self):
        return self._trim(self.staled_gradients_remote_padded())

    def staled_gradients_local(self):
        return self._trim(self.staled_gradients_local_padded())
