"""EmbCache: an HBM-resident hot-row cache in front of a cold table (device or pinned host).

Host-side mirror of the reference's LocalSparseAdamStateCache (python/EmbCache/cache.py:34-199):
same hotness placement (create_cache, :133-194), same __getitem__/__setitem__ contract (:66-131),
but keyed by the ascending hot-ID set and a binary search instead of a dense index_map over all
rows (88.8 MB instead of 888 MB at 111 M rows), and with the lookup fused into the row kernels.
"""
import torch

from . import EmbCacheLib, ops


def select_hot_ids(hotness, num_hot, candidate_ids=None):
    """The reference's placement rule (python/EmbCache/cache.py:165-168): the `num_hot` candidates
    with the largest hotness, ties in argsort order; returned sorted ascending (int64, CPU)."""
    hotness = torch.as_tensor(hotness)
    if candidate_ids is None:
        candidate_ids = torch.arange(hotness.numel(), dtype=torch.int64)
    order = torch.argsort(hotness[candidate_ids], descending=True)
    chosen = candidate_ids[order][:num_hot]
    return torch.sort(chosen.to(torch.int64)).values


def hot_ids_by_threshold(hotness, hot_threshold):
    """ids with hotness >= hot_threshold, ascending (python/EmbCache/dist_emb.py:109)."""
    return torch.nonzero(torch.as_tensor(hotness) >= hot_threshold).flatten().to(torch.int64)


class EmbCache:
    """Hot cache over one or more row tables that share the same row ids.

    cold_tables : list of [N, D_k] (or [N]) tensors, on the device or pinned on the host.
    hot_ids     : ascending duplicate-free int64 ids of the cached rows.
    The hot copies are gathered from the cold tables at construction; afterwards the hot copy is
    the live one for cached rows (writes go to it only), as in the reference (cache.py:113-121).
    """

    def __init__(self, cold_tables, hot_ids, device="cuda", count_hit=False):
        self.device = torch.device(device)
        self.cold = list(cold_tables)
        hot_ids = torch.as_tensor(hot_ids, dtype=torch.int64)
        if hot_ids.numel() > 1:
            assert bool((hot_ids[1:] > hot_ids[:-1]).all()), "hot_ids must be ascending and unique"
        self.hot_ids = hot_ids.to(self.device)
        self.hot_set = ops.HotSet(self.hot_ids)
        self.hot = []
        for t in self.cold:
            if t.is_cuda:
                self.hot.append(t[self.hot_ids].contiguous())
            else:
                # a pinned host table is read zero-copy by the gather kernel, not indexed on the CPU
                hot = torch.empty((self.hot_ids.numel(),) + tuple(t.shape[1:]), dtype=t.dtype,
                                  device=self.device)
                if t.dtype in (torch.float32, torch.float64):
                    EmbCacheLib.cudaFetch2(t, self.hot_ids, hot)
                else:
                    hot.copy_(t[hot_ids.cpu()])
                self.hot.append(hot)
        self.num_rows = self.cold[0].size(0)
        self._count_hit = count_hit
        self._hit_num = 0
        self._lookup_num = 0

    @classmethod
    def create_cache(cls, cold_tables, hotness, alloca_mem_size, device="cuda", **kw):
        """Budgeted placement as in python/EmbCache/cache.py:133-194: the id set costs 8 bytes per
        cached row (not per table row), each cached row costs its bytes in every table."""
        item = sum(t.element_size() * (t[0].numel() if t.dim() > 1 else 1) for t in cold_tables) + 8
        cached_num = int(min(max(alloca_mem_size, 0) // item, cold_tables[0].size(0)))
        return cls(cold_tables, select_hot_ids(hotness, cached_num), device=device, **kw)

    # -- the operators ---------------------------------------------------------
    def lookup(self, ids):
        return ops.lookup(ids, self.hot_set)

    def split(self, ids):
        """(hot_mask, hot_pos, cold_pos) of a query batch; one host synchronisation."""
        return ops.split(self.lookup(ids))

    def cached_fetch(self, ids, table=0, out=None):
        if self._count_hit:
            self._hit_num += int((self.lookup(ids) >= 0).sum().item())
            self._lookup_num += ids.numel()
        return ops.cached_fetch(self.cold[table], self.hot[table], ids, self.hot_set, out=out)

    def cached_set(self, ids, rows, table=0):
        ops.cached_set(rows, self.cold[table], self.hot[table], ids, self.hot_set)

    def __getitem__(self, ids):
        return tuple(self.cached_fetch(ids, k) for k in range(len(self.cold)))

    def __setitem__(self, ids, values):
        for k, v in enumerate(values):
            self.cached_set(ids, v, k)

    def get_hit_rate(self):
        return 0 if self._lookup_num == 0 else self._hit_num / self._lookup_num

    def write_back(self):
        """Copies the hot rows back into the cold tables (e.g. before saving them)."""
        for cold, hot in zip(self.cold, self.hot):
            if cold.is_cuda:
                cold[self.hot_ids] = hot
            elif cold.dtype in (torch.float32, torch.float64):
                EmbCacheLib.cudaSet(hot, cold, self.hot_ids)     # scatter into the pinned table
                torch.cuda.current_stream().synchronize()        # the host may read it next
            else:
                cold[self.hot_ids.cpu()] = hot.cpu()
