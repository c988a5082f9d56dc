"""DistEmb on one GPU: the reference's embedding module and its sparse optimizers over the keyed
schedule of this build.

Mirrors python/EmbCache/dist_emb.py (DistEmb :11-52, DistEmbeddingTensor :55-292) and the
optimizer front end of python/EmbCache/sparse_optim.py (DistembSparseGradOptimizer.step :212-445,
SparseAdam :531-590) for a single trainer: the forward call records (ids, rows, plan) in the
embedding's `trace` exactly where the reference appends to it (:276-288), and `optimizer.step()`
consumes the trace (:225-238).  What lies between a trainer and its partition in the reference -
the DGL DistTensor, the cache server and its client, the cross-trainer exchange - is not part of
this build; the table is one tensor on this GPU's host (page-locked, read and written zero-copy)
or in its HBM, and the hot rows are the ids whose hotness reaches `hot_threshold` (:109).

    emb = DistEmb(num_nodes, dim, torch.float32, "emb", hotness_list=hotness, hot_threshold=150)
    opt = SparseAdam([emb.sparse_emb], lr=0.01)
    rows = emb(ids)                  # lookup + hot/cold split + both gathers + sort of the keys
    loss(model(rows)).backward()
    opt.step()                       # segmented sums, mean over duplicate ids, fused row updates
"""
import torch
import torch.nn as nn

from . import cache as _cache
from . import ops
from . import sparse_optim as _engine


def tensor_initializer(shape, dtype):
    """python/EmbCache/common.py:13-16."""
    tensor = torch.zeros(shape, dtype=dtype)
    tensor.uniform_(-1, 1)
    return tensor


class DistEmbeddingTensor:
    """The sparse embedding behind DistEmb (python/EmbCache/dist_emb.py:55-292), one trainer.

    Arguments keep the reference's names and order; the ones that describe other trainers and the
    cache server (local_rank, local_trainer_num, part_book, cache_server_addr, cache_server_port)
    are accepted and must describe a single trainer.  Keyword-only additions: `weight` (initial
    table instead of tensor_initializer), `pin_memory` (True: the table lives in page-locked host
    memory like the reference's pinned partition, :79-81; False: in HBM), `device`.
    """

    def __init__(self, num_nodes, emb_dim, emb_dtype, name, cache_rate=0.3, idx_dtype=None,
                 local_rank=None, local_trainer_num=None, hotness_list=None, hot_threshold=150,
                 part_book=None, cache_server_addr=None, cache_server_port=None, *, weight=None,
                 pin_memory=True, device="cuda"):
        if emb_dtype != torch.float32:
            raise RuntimeError("DistEmbeddingTensor: the row optimizers work in float32")
        if local_trainer_num not in (None, 1) or local_rank not in (None, 0):
            raise RuntimeError("this build runs one trainer: local_rank 0 of 1")
        self.name = name
        self.num_embeddings = int(num_nodes)
        self.embedding_dim = int(emb_dim)
        self._emb_dtype = emb_dtype
        self._idx_dtype = idx_dtype
        self._device = torch.device(device)
        table = weight if weight is not None else tensor_initializer((num_nodes, emb_dim), emb_dtype)
        if tuple(table.shape) != (num_nodes, emb_dim):
            raise RuntimeError("weight must be [num_nodes, emb_dim]")
        if pin_memory:
            self.tensor = table if (not table.is_cuda and table.is_pinned()) else table.cpu().pin_memory()
        else:
            self.tensor = table.to(self._device)
        self.enable_cache = cache_rate > 0
        if self.enable_cache:
            assert hotness_list is not None
            self._hotness = torch.as_tensor(hotness_list)
            # hot = hotness >= hot_threshold (:109), at most cache_rate * num_nodes of them, the
            # hottest first (the placement rule of python/EmbCache/cache.py:165-168)
            hot = _cache.hot_ids_by_threshold(self._hotness, hot_threshold)
            cap = int(num_nodes * cache_rate)
            if hot.numel() > cap:
                hot = _cache.select_hot_ids(self._hotness, cap, candidate_ids=hot)
            self.hot_ids = hot
        else:
            self.hot_ids = torch.empty(0, dtype=torch.int64)
        self._plain = None          # hot copy for fetches before an optimizer is attached
        self._opt = None            # the row optimizer that owns hot copies and state
        self.trace = []

    # -- the optimizer attaches itself: from then on its tables are the live ones ----------------
    def _attach(self, row_optimizer):
        self._opt = row_optimizer
        self._plain = None

    def _fetch_only(self, ids):
        if self._opt is not None:
            return ops.cached_fetch(self._opt.cold_w, self._opt.hot_w, ids, self._opt.hot_set) \
                if self._opt.cold_w.is_contiguous() else self._opt.fetch_split(ids)
        if self._plain is None:
            self._plain = _cache.EmbCache([self.tensor], self.hot_ids, device=self._device)
        return self._plain.cached_fetch(ids)

    def __call__(self, ids, device=torch.device("cuda"), is_training=True):
        ids = ids.to(self._device)
        if ids.dtype != torch.int64:
            ids = ids.long()
        if not is_training:
            return self._fetch_only(ids)
        state = None
        if self._opt is not None and torch.is_grad_enabled():
            emb, state = self._opt.forward_keyed(ids)
        else:
            emb = self._fetch_only(ids)
        emb.requires_grad_(True)
        emb.retain_grad()
        if torch.is_grad_enabled():
            self.trace.append((ids, emb, state))
        return emb

    def reset_trace(self):
        """Reset the traced data (python/EmbCache/dist_emb.py:290-292)."""
        self.trace = []

    def weight_rows(self, ids):
        """Current rows of `ids` (hot copy if hot, else the table): for inspection and saving."""
        return self._fetch_only(ids.to(self._device).long())


class DistEmb(nn.Module):
    """python/EmbCache/dist_emb.py:11-52."""

    def __init__(self, num_nodes, emb_dim, emb_dtype, name, cache_rate=0.3, idx_dtype=None,
                 local_rank=None, local_trainer_num=None, hotness_list=None, hot_threshold=150,
                 part_book=None, cache_server_addr=None, cache_server_port=None, **kw):
        super().__init__()
        self.emb_dim = emb_dim
        self.sparse_emb = DistEmbeddingTensor(
            num_nodes, emb_dim, emb_dtype, name, cache_rate=cache_rate, idx_dtype=idx_dtype,
            local_rank=local_rank, local_trainer_num=local_trainer_num, hotness_list=hotness_list,
            hot_threshold=hot_threshold, part_book=part_book, cache_server_addr=cache_server_addr,
            cache_server_port=cache_server_port, **kw)
        self._device = torch.device(kw.get("device", "cuda"))

    def forward(self, idx):
        return self.sparse_emb(idx, self._device, self.training)

    def timecheck(self):
        pass


class DistembSparseGradOptimizer:
    """Front end of the sparse optimizers (python/EmbCache/sparse_optim.py:160-445), one trainer:
    step() takes every embedding's trace - the ids and rows of its forward calls since the last
    step - and applies one update per distinct id with the MEAN of its gradient rows, as the
    reference's update does (unique_grads, :142-157, called at :613).  One forward call per step
    runs the keyed schedule (the plan made at forward time, segmented sums and fused row updates,
    the cold update reusing the forward rows); several calls are concatenated first, like :225-238,
    and go through the split schedule."""

    def __init__(self, params, lr, num_parts=1, local_group=None, partition_group=None):
        if num_parts not in (None, 1):
            raise RuntimeError("this build runs one partition")
        self._params = list(params)
        self._lr = lr
        self._clean_grad = False
        self._state = {}
        for emb in self._params:
            assert emb.name not in self._state, "{} already registered in the optimizer".format(emb.name)
            row_opt = self._make_row_optimizer(emb)
            self._state[emb.name] = row_opt
            emb._attach(row_opt)

    def _make_row_optimizer(self, emb):
        raise NotImplementedError

    def step(self):
        with torch.no_grad():
            for emb in self._params:
                row_opt = self._state[emb.name]
                trace = [t for t in emb.trace if t[1].grad is not None]
                if len(trace) == 1 and trace[0][2] is not None:
                    ids, rows, state = trace[0]
                    row_opt.backward_keyed(state, rows.grad, average="mean")
                elif trace:
                    idics = torch.cat([t[0] for t in trace], dim=0)
                    grads = torch.cat([t[1].grad for t in trace], dim=0)
                    row_opt.step_split(idics, grads.contiguous(), average="mean")
                emb.reset_trace()

    def zero_grad(self):
        """clean grad cache (python/EmbCache/sparse_optim.py:468-470): the traced rows and their
        gradients are dropped with the trace at the end of step()."""
        self._clean_grad = True


class SparseAdam(DistembSparseGradOptimizer):
    """python/EmbCache/sparse_optim.py:531-590 (constructor) and :590-685 (update) over the fused
    row kernels.  `state_on_device` keeps step / mem / power of the cold rows in HBM even when
    the table is in host memory."""

    def __init__(self, params, lr, num_parts=1, local_group=None, partition_group=None,
                 betas=(0.9, 0.999), eps=1e-08, state_on_device=False):
        self._beta1, self._beta2, self._eps = betas[0], betas[1], eps
        self._state_on_device = state_on_device
        self._defaults = {"_lr": lr, "_eps": eps, "_beta1": betas[0], "_beta2": betas[1]}
        super().__init__(params, lr, num_parts, local_group, partition_group)

    def _make_row_optimizer(self, emb):
        return _engine.SparseAdam(emb.tensor, emb.hot_ids, lr=self._lr, betas=(self._beta1, self._beta2),
                                  eps=self._eps, device=emb._device,
                                  state_on_device=self._state_on_device)


class SparseAdagrad(DistembSparseGradOptimizer):
    """The same front end over sparse Adagrad, the optimizer of the benchmark configurations
    (absent from the reference, whose only optimizer is SparseAdam)."""

    def __init__(self, params, lr, num_parts=1, local_group=None, partition_group=None, eps=1e-10,
                 state_on_device=False):
        self._eps = eps
        self._state_on_device = state_on_device
        self._defaults = {"_lr": lr, "_eps": eps}
        super().__init__(params, lr, num_parts, local_group, partition_group)

    def _make_row_optimizer(self, emb):
        return _engine.SparseAdagrad(emb.tensor, emb.hot_ids, lr=self._lr, eps=self._eps,
                                     device=emb._device, state_on_device=self._state_on_device)
