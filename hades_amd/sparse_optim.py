"""Gradient combine and sparse row optimizers, host side.

Mirrors the reference's python/EmbCache/sparse_optim.py for one GPU: `only_unique_grads` and
`unique_grads` keep the reference's names, arguments and return values (:132-157); SparseAdagrad
(the optimizer of the benchmark configurations) and SparseAdam (the one the reference ships,
:531-685) run the whole update - lookup, state gather, row math, scatter-back - in one kernel over
an EmbCache-style (hot, cold) table pair.  The cross-trainer all-to-all of the reference
(:19-129, 267-341) is not part of this build.
"""
import os
import warnings
import weakref

import torch

from . import EmbCacheLib, ops


def bucket_gradients(idics, grads, partition_range, num_parts, num_trainers_per_part,
                     grads_cnt=None):
    """The part of swap_gradients that precedes its all-to-all (python/EmbCache/sparse_optim.py:
    33-62), argument names as there: ids, gradient rows and counts grouped by owning trainer, and
    the per-trainer row counts.  Returns (ids, grads, grads_cnt, input_splits_tensor) with
    input_splits_tensor int64[num_parts * num_trainers_per_part] on the device (the reference
    then calls .tolist() on it for the exchange, :52)."""
    num_owners = int(num_parts * num_trainers_per_part)
    return ops.bucket_by_owner(idics, grads, grads_cnt, partition_range,
                               int(num_trainers_per_part), num_owners)


def only_unique_grads(idx, grad, id_bound=0, mode=ops.COMBINE_FAST):
    """(unique ids ascending, per-id summed float32 grads, per-id counts) - python/EmbCache/sparse_optim.py:132-139."""
    return ops.combine(idx, grad, id_bound=id_bound, mode=mode)


def unique_grads(idx, grad, cnt=None, id_bound=0, mode=ops.COMBINE_FAST):
    """(unique ids, per-id mean grads) - python/EmbCache/sparse_optim.py:142-157.

    With `cnt` given, the divisor of row u is 1 + sum of the cnt entries of its occurrences: the
    reference starts that count from ones (:145-148) and this keeps it."""
    if cnt is None:
        uids, sums, cnts, nu = ops.combine_padded(idx, grad, id_bound, mode)
        ops.rows_div_count_(sums, cnts, nu)
        u = int(nu.item())
        if u < 0:
            raise ops._bound_error()
        return uids[:u], sums[:u]
    uids, sums, _, nu, inverse = ops.combine_padded(idx, grad, id_bound, mode, return_inverse=True)
    u = int(nu.item())
    if u < 0:
        raise ops._bound_error()
    grad_cnt = torch.ones(u, dtype=cnt.dtype, device=cnt.device)
    grad_cnt.index_add_(0, inverse.long(), cnt)
    sums = sums[:u] / grad_cnt.unsqueeze(1)
    return uids[:u], sums


_side_streams = {}


def side_stream(device, k):
    """The k-th (0, 1, 2) side stream of this module on `device`, created once per process and
    shared by every optimizer: HIP serves a process's streams from a handful of hardware queues
    (four by default), and streams that share a queue run one after the other, so a process
    that wants its cold, prefetch and sort streams to overlap with its main stream must not
    create a fresh set per optimizer."""
    key = (torch.device(device).index or 0, int(k))
    if key not in _side_streams:
        _check_hw_queues()
        _side_streams[key] = torch.cuda.Stream(device=device)
    return _side_streams[key]


_hw_queues_checked = False


def _check_hw_queues():
    """The schedules here are built for HIP's default of four hardware queues per process (the
    caller's stream and three side streams).  A process that ran them with GPU_MAX_HW_QUEUES=8
    died with a segmentation fault when copies were first issued on the side streams; the cause
    is not known, so a raised limit is reported instead of being used silently."""
    global _hw_queues_checked
    if _hw_queues_checked:
        return
    _hw_queues_checked = True
    v = os.environ.get("GPU_MAX_HW_QUEUES")
    try:
        if v is not None and int(v) > 4:
            warnings.warn("GPU_MAX_HW_QUEUES=%s: hades_amd's multi-stream schedules are validated with "
                          "the default of 4 hardware queues only; a run with 8 ended in a segmentation "
                          "fault of unknown cause.  Unset the variable." % v, RuntimeWarning, stacklevel=3)
    except ValueError:
        pass


class _SparseRowOptimizer:
    """State shared by the two optimizers: weights and state as (hot, cold) pairs keyed by the
    ascending hot-ID set.  `weight_cold` is [N, D] on the device or pinned on the host."""

    def __init__(self, weight_cold, hot_ids, lr, device="cuda", state_on_device=False,
                 reuse_fetched_rows=True):
        self.device = torch.device(device)
        # backward_keyed may take the old cold weights from the rows forward_keyed fetched instead
        # of reading the cold table a second time.  That is right only while nothing has written
        # the table in between: every update this optimizer issues bumps `_epoch`, the forward
        # state carries the epoch (and torch's version counters of the table and of the rows), and
        # the backward half reuses the rows only if all of them are unchanged.  Writers this
        # object cannot see (another optimizer or a raw kernel on the same table) either call
        # note_table_write() or construct with reuse_fetched_rows=False.
        self.reuse_fetched_rows = bool(reuse_fetched_rows)
        self._epoch = 0
        self._rows_writer = {}      # storage address -> plan of the forward half that last wrote it
        # cold optimizer state normally lives where the cold weights live; with state_on_device
        # it is kept in HBM even when the weights are a pinned host table (288 GB of HBM hold the
        # state of tables whose weights are served from the host)
        self.state_on_device = state_on_device
        self.lr = lr
        self.cold_w = weight_cold
        self.num_rows, self.dim = weight_cold.shape
        hot_ids = torch.as_tensor(hot_ids, dtype=torch.int64)
        self.hot_ids = hot_ids.to(self.device)
        self.hot_set = ops.HotSet(self.hot_ids)
        self.hot_w = self._gather_hot(weight_cold)
        self._ws = ops.Workspace(self.device)
        self._side = None
        self._kbufs = {}            # buffer sets of the keyed steps, by slot

    def _gather_hot(self, cold):
        """Hot copy of the rows named by hot_ids; a pinned host table is read zero-copy by the
        gather kernel instead of being indexed on the CPU."""
        if cold.is_cuda:
            return cold[self.hot_ids].contiguous()
        h = self.hot_ids.numel()
        out = torch.empty((h,) + tuple(cold.shape[1:]), dtype=cold.dtype, device=self.device)
        if cold.is_contiguous():
            EmbCacheLib.cudaFetch2(cold, self.hot_ids, out)
        elif h:                                   # row-strided host table
            ops.fetch_listed(cold, self.hot_ids, torch.arange(h, device=self.device),
                             torch.tensor([h], dtype=torch.int64, device=self.device), out)
        return out

    def _new_state_like(self, cold, shape=None):
        shape = shape or tuple(cold.shape)
        if cold.is_cuda or self.state_on_device:
            return torch.zeros(shape, dtype=torch.float32, device=self.device)
        t = torch.empty(shape, dtype=torch.float32, pin_memory=True)
        # zero it from the device in slices (a 57 GB memset on one host core takes far longer)
        flat = t.view(-1)
        step = 1 << 28
        zeros = torch.zeros(min(step, flat.numel()), dtype=torch.float32, device=self.device)
        for i in range(0, flat.numel(), step):
            m = min(step, flat.numel() - i)
            flat[i:i + m].copy_(zeros[:m])
        return t

    def note_table_write(self):
        """Tells the optimizer that its tables were written by something it did not launch (a raw
        kernel, another object sharing the tables): rows fetched before this call are no longer
        trusted as the old weights of a later backward_keyed."""
        self._epoch += 1

    def _table_stamp(self):
        """What must be unchanged between a forward fetch and the reuse of its rows: this
        optimizer's own update count and torch's in-place version counter of the cold table."""
        return (self._epoch, self.cold_w._version)

    def _stamp_forward(self, plan, rows, stamp=None):
        plan.rows = rows
        plan.rows_version = rows._version
        plan.table_stamp = self._table_stamp() if stamp is None else stamp
        # a later forward half that writes into the same storage (through raw pointers: no version
        # bump) takes the rows away from this plan
        dead = [k for k, r in self._rows_writer.items() if r() is None]
        for k in dead:
            del self._rows_writer[k]
        self._rows_writer[rows.untyped_storage().data_ptr()] = weakref.ref(plan)

    def _rows_to_reuse(self, plan, fetched_rows):
        """The rows the cold update may take its old weights from, or None (read the table).
        fetched_rows: "auto" (the guarded default), None (never), or a tensor the caller vouches
        for."""
        if fetched_rows is None:
            return None
        if not isinstance(fetched_rows, str):
            return fetched_rows
        if fetched_rows != "auto":
            raise RuntimeError("fetched_rows must be 'auto', None or a tensor")
        rows = getattr(plan, "rows", None)
        if (not self.reuse_fetched_rows or rows is None or getattr(plan, "first_pos", None) is None
                or plan.table_stamp != self._table_stamp() or plan.rows_version != rows._version
                or self._rows_writer.get(rows.untyped_storage().data_ptr(), lambda: None)() is not plan):
            return None
        return rows

    def fetch(self, ids, out=None):
        """Forward fetch of embedding rows (cached_fetch)."""
        return ops.cached_fetch(self.cold_w, self.hot_w, ids, self.hot_set, out=out)

    def prepare(self, idx, stream=None, out=None):
        """Starts the id-only half of the next step's combine (sort + run boundaries) on a side
        stream and returns its plan.  The ids of a batch are known at forward time - the reference
        saves them in its trace (python/EmbCache/dist_emb.py:276-288) - so this work can hide
        behind the fetch and the model's forward/backward; step(..., plan=plan) waits for it.
        One plan may be outstanding per optimizer (it lives in the optimizer's workspace)."""
        cur = torch.cuda.current_stream()
        if out is None:   # allocated on the caller's stream, which is where they are consumed
            out = (torch.empty(idx.numel(), dtype=torch.int64, device=self.device),
                   torch.empty(1, dtype=torch.int64, device=self.device))
        if stream is None:
            if self._side is None:
                self._side = side_stream(self.device, 2)
            stream = self._side
        # everything queued so far (the ids, and the previous step that used the workspace) first
        stream.wait_stream(cur)
        with torch.cuda.stream(stream):
            plan = ops.combine_plan(idx, self.dim, id_bound=self.num_rows, workspace=self._ws,
                                    out=out)
            plan.ready = torch.cuda.Event()
            plan.ready.record(stream)
        return plan

    # ---- the split schedule: hot rows and cold rows on separate kernels and streams ----------
    # The reference's forward path splits a batch by class first and then gathers per class
    # (python/EmbCache/dist_emb.py:174-211).  Here: one lookup + stable partition, then the hot
    # positions go through kernels that only touch HBM while the cold positions go through
    # kernels that only touch the host table, on a second stream of the same priority, so the
    # host-link time and the HBM time overlap instead of adding up.
    # one_stream = True runs the cold class on the caller's stream too (no overlap): the same
    # kernels one after the other, e.g. to time each of them undisturbed
    one_stream = False
    # backward_keyed: the cold update sums the gradient rows of its runs itself instead of waiting
    # for a segmented sum of the cold class (False: segmented-sum kernels first, as for the hot class)
    fuse_cold_sums = True
    # width (workgroups) of a write-only cold update that runs beside a prefetched gather.  cfg3,
    # two batches in flight, gather 16 blocks: update 32 / 64 blocks wide -> step 1.31 / 1.43 ms
    # (gather 1.12 / 0.99 ms, update 1.14 / 1.06 ms: what one direction gains the other loses)
    pipelined_update_blocks = 32

    def _split_state(self):
        if getattr(self, "_cold_stream", None) is None:
            self._cold_stream = side_stream(self.device, 0)
            self._split_bufs = {}
            self._split_ws = ops.Workspace(self.device)
            self._cold_done = None
        return torch.cuda.current_stream() if self.one_stream else self._cold_stream

    def _split_out(self, key, n):
        bufs = self._split_bufs.get(key)
        if bufs is None or bufs[0].numel() < n:
            dev = self.device
            bufs = (torch.empty(n, dtype=torch.int64, device=dev), torch.empty(n, dtype=torch.int64, device=dev),
                    torch.empty(n, dtype=torch.int64, device=dev), torch.empty(2, dtype=torch.int64, device=dev))
            self._split_bufs[key] = bufs
        return bufs

    def join(self):
        """Makes torch's current stream wait for everything queued on the cold stream."""
        if getattr(self, "_cold_done", None) is not None:
            torch.cuda.current_stream().wait_event(self._cold_done)
            self._cold_done = None

    @staticmethod
    def _timed(timing, name, stream, fn):
        """Runs fn(); with timing = {name: (start, stop)} (torch events, enable_timing=True) the
        pair is recorded on `stream` right before and after it."""
        pair = timing.get(name) if timing else None
        if pair:
            pair[0].record(stream)
        fn()
        if pair:
            pair[1].record(stream)

    def fetch_split(self, ids, out=None, join=True, timing=None):
        """cached_fetch as lookup -> stable hot/cold partition -> one gather per class: the hot
        class from the HBM copy on the current stream, the cold class from the cold table on the
        cold stream.  With join=False the caller calls join() before anything reads `out` or
        writes the tables on the current stream.  `timing` may map "hot_fetch" / "cold_fetch" to
        event pairs that are recorded around the two gather kernels on their streams."""
        cold = self._split_state()
        cur = torch.cuda.current_stream()
        n = ids.numel()
        if out is None:
            out = torch.empty((n, self.dim), dtype=self.hot_w.dtype, device=self.device)
        loc, hot_pos, cold_pos, counts = ops.lookup_split(
            ids, self.hot_set, workspace=self._split_ws, out=self._split_out("fetch", n))
        hot_pos, cold_pos = hot_pos[:n], cold_pos[:n]
        split_done = torch.cuda.Event()
        split_done.record(cur)
        cold.wait_event(split_done)
        if cold != cur:       # memory of the caller's stream, used on another one
            out.record_stream(cold)
            ids.record_stream(cold)
        with torch.cuda.stream(cold):
            self._timed(timing, "cold_fetch", cold,
                        lambda: ops.fetch_listed(self.cold_w, ids, cold_pos, counts[1:2], out))
            self._cold_done = torch.cuda.Event()
            self._cold_done.record(cold)
        if self.hot_ids.numel():
            self._timed(timing, "hot_fetch", cur,
                        lambda: ops.fetch_listed(self.hot_w, loc, hot_pos, counts[0:1], out))
        if join:
            self.join()
        return out

    def _update_class(self, index, grad, pos, count, hot):
        raise NotImplementedError

    def update_split(self, uids, grad, num_unique=None, join=True, timing=None, cnts=None,
                     average=None):
        """The row update over a combined batch as lookup -> partition -> one update kernel per
        class, hot on the current stream and cold on the cold stream ("hot_update" /
        "cold_update" in `timing`).  `average` = "mean" / "one_plus" with `cnts` (the combine's
        counts) divides the rows of `grad` in place by their counts (plus one) first: the
        reference's unique_grads (python/EmbCache/sparse_optim.py:142-157)."""
        cold = self._split_state()
        cur = torch.cuda.current_stream()
        n = uids.numel()
        if ops._average_code(average):
            if cnts is None:
                raise RuntimeError("update_split(average=...) needs the combine's cnts")
            ops.rows_div_count_(grad, cnts, num_unique, one_plus=average == "one_plus")
        loc, hot_pos, cold_pos, counts = ops.lookup_split(
            uids, self.hot_set, num_live=num_unique, workspace=self._split_ws,
            out=self._split_out("update", n))
        hot_pos, cold_pos = hot_pos[:n], cold_pos[:n]
        split_done = torch.cuda.Event()
        split_done.record(cur)
        cold.wait_event(split_done)          # the cold stream also still orders after its own fetch
        self._epoch += 1
        if cold != cur:       # memory of the caller's stream, read on another one
            for t in (uids, grad, num_unique):
                if t is not None:
                    t.record_stream(cold)
        with torch.cuda.stream(cold):
            self._timed(timing, "cold_update", cold,
                        lambda: self._update_class(uids, grad, cold_pos, counts[1:2], hot=False))
            self._cold_done = torch.cuda.Event()
            self._cold_done.record(cold)
        if self.hot_ids.numel():
            self._timed(timing, "hot_update", cur,
                        lambda: self._update_class(loc, grad, hot_pos, counts[0:1], hot=True))
        if join:
            self.join()

    # ---- the keyed step: one lookup per query serves the gather, the combine and the update ----
    def forward_keyed(self, ids, out=None, timing=None, bufs=None, slot=None):
        """Forward half of a training step on the split schedule.  One lookup gives every query
        its slot, its class list and a class-ordered sort key; the hot rows are gathered on the
        current stream and the cold rows on the cold stream; meanwhile the keys are sorted (the
        id-only half of the combine).  Returns (rows, state) after joining the two streams: the
        rows are complete, `state` goes to backward_keyed with the gradients."""
        cold = self._split_state()
        cur = torch.cuda.current_stream()
        n = ids.numel()
        if out is None:
            out = torch.empty((n, self.dim), dtype=self.hot_w.dtype, device=self.device)
        kb = ops.key_bits_for(max(self.num_rows, self.hot_ids.numel(), 2))
        if bufs is None:      # slot: see prefetch_keyed (the first batch of a pipelined run)
            bufs = self._keyed_bufs(n, slot)
        loc, hot_pos, cold_pos, counts = ops.lookup_split(
            ids, self.hot_set, workspace=bufs.get("split_ws", self._split_ws), out=bufs["split"],
            sort_keys=bufs["keys"], key_bits=kb)
        hot_pos, cold_pos = hot_pos[:n], cold_pos[:n]
        split_done = torch.cuda.Event()
        split_done.record(cur)
        cold.wait_event(split_done)
        if cold != cur:       # memory of the caller's stream, used on another one
            out.record_stream(cold)
            ids.record_stream(cold)
        with torch.cuda.stream(cold):
            self._timed(timing, "cold_fetch", cold,
                        lambda: ops.fetch_listed(self.cold_w, ids, cold_pos, counts[1:2], out))
            self._cold_done = torch.cuda.Event()
            self._cold_done.record(cold)
        if self.hot_ids.numel():
            self._timed(timing, "hot_fetch", cur,
                        lambda: ops.fetch_listed(self.hot_w, loc, hot_pos, counts[0:1], out))
        plan = ops.combine_plan_classed(bufs["keys"][:n], self.dim, kb, workspace=bufs.get("ws", self._ws),
                                        out=(bufs["ukeys"][:n], bufs["nu"], bufs["class_split"]),
                                        first_pos=bufs["first_pos"][:n])
        self._stamp_forward(plan, out)
        self.join()
        return out, (plan, bufs)

    def _keyed_bufs(self, n, slot=None):
        """Buffers of one keyed step.  slot = None: the optimizer's single set, with the shared
        workspaces (one batch in flight).  slot = 0 / 1: one of two sets that also own their
        workspaces, for the pipelined schedule where two batches are in flight."""
        sets = self._kbufs
        b = sets.get(slot)
        if b is None or b["keys"].numel() < n:
            dev = self.device
            if b is not None:
                # a larger batch: the old set may still be read on a side stream, and the caching
                # allocator hands freed blocks back without asking the side streams
                torch.cuda.synchronize(dev)
            i64 = lambda k: torch.empty(k, dtype=torch.int64, device=dev)
            b = {"split": (i64(n), i64(n), i64(n), i64(2)), "keys": i64(n), "ukeys": i64(n),
                 "nu": i64(1), "class_split": i64(2),
                 "first_pos": torch.empty(n, dtype=torch.int32, device=dev),
                 "sums": torch.empty((n, self.dim), dtype=torch.float32, device=dev), "cnts": i64(n)}
            if slot is not None:
                b["ws"], b["split_ws"] = ops.Workspace(dev), ops.Workspace(dev)
            sets[slot] = b
        return b

    # ---- the pipelined keyed step: the next batch's cold rows cross the host link while the
    # ---- current batch's cold update writes the table ------------------------------------------
    # The link carries reads and writes at the same time, and a keyed step uses one direction at a
    # time for most of its length (gather: reads; update with fetched_rows: writes).  A trainer
    # that has the ids of batch i+1 before the backward half of batch i (the reference's sampler
    # runs ahead of the step) calls
    #     p = opt.prefetch_keyed(ids_next, slot=(i + 1) % 2, out=rows_next)
    #     opt.backward_keyed(state_i, grads_i, fetched_rows=rows_i, join=False)
    #     rows_next, state_next = opt.finish_prefetch(p, after=state_i)
    # and gets, bit for bit, the rows and tables of the one-batch-at-a-time order: the rows that
    # batch i's update wrote (its distinct cold ids; usually a handful of the next batch's) are
    # read again after that update, the hot rows are gathered after the hot update as before.
    def prefetch_keyed(self, ids, slot, out=None, timing=None):
        """Starts the forward half of the NEXT batch on side streams: lookup + partition + cold
        gather on one, the sort of the class-ordered keys on another.  Nothing of it is visible to
        the caller's stream until finish_prefetch.  `slot` (0 or 1) alternates from batch to
        batch; `out` must not be the rows buffer of the batch whose backward half is pending."""
        self._split_state()
        if getattr(self, "_pre_stream", None) is None:
            self._pre_stream = side_stream(self.device, 1)
            self._sort_stream = side_stream(self.device, 2)
        cur, pre, srt = torch.cuda.current_stream(), self._pre_stream, self._sort_stream
        n = ids.numel()
        if out is None:
            out = torch.empty((n, self.dim), dtype=self.hot_w.dtype, device=self.device)
        kb = ops.key_bits_for(max(self.num_rows, self.hot_ids.numel(), 2))
        bufs = self._keyed_bufs(n, slot)
        pre.wait_stream(cur)      # the ids, and everything that last used this slot's buffers
        out.record_stream(pre)    # memory of the caller's stream, used on another one
        ids.record_stream(pre)
        with torch.cuda.stream(pre):
            loc, hot_pos, cold_pos, counts = ops.lookup_split(
                ids, self.hot_set, workspace=bufs["split_ws"], out=bufs["split"],
                sort_keys=bufs["keys"], key_bits=kb)
            looked_up = torch.cuda.Event()
            looked_up.record(pre)
            self._timed(timing, "cold_fetch", pre,
                        lambda: ops.fetch_listed(self.cold_w, ids, cold_pos[:n], counts[1:2], out))
            gathered = torch.cuda.Event()
            gathered.record(pre)
        srt.wait_event(looked_up)
        with torch.cuda.stream(srt):
            plan = ops.combine_plan_classed(bufs["keys"][:n], self.dim, kb, workspace=bufs["ws"],
                                            out=(bufs["ukeys"][:n], bufs["nu"], bufs["class_split"]),
                                            first_pos=bufs["first_pos"][:n])
            planned = torch.cuda.Event()
            planned.record(srt)
        self._prefetching = True
        return {"ids": ids, "out": out, "plan": plan, "bufs": bufs, "loc": loc, "hot_pos": hot_pos[:n],
                "cold_pos": cold_pos[:n], "counts": counts, "looked_up": looked_up,
                "gathered": gathered, "planned": planned, "stamp": self._table_stamp()}

    def finish_prefetch(self, p, after=None, timing=None):
        """Completes a prefetched forward half on the current stream, after the backward half of
        the batch before it (`after` = that batch's state, or None if there was none) has been
        queued: gathers the hot rows (behind the hot update), waits for the cold update, re-reads
        the cold rows that update wrote, and returns (rows, state) like forward_keyed."""
        cur = torch.cuda.current_stream()
        ids, out, counts = p["ids"], p["out"], p["counts"]
        self._prefetching = False
        cur.wait_event(p["looked_up"])
        if self.hot_ids.numel():
            self._timed(timing, "hot_fetch", cur,
                        lambda: ops.fetch_listed(self.hot_w, p["loc"], p["hot_pos"], counts[0:1], out))
        self.join()                         # the cold update of the batch before
        cur.wait_event(p["gathered"])
        if after is not None:
            prev = after[0]
            self._timed(timing, "cold_refresh", cur,
                        lambda: ops.fetch_listed(self.cold_w, ids, p["cold_pos"], counts[1:2], out,
                                                 only_in=prev.uids, only_in_count=prev.class_split[1:2]))
        cur.wait_event(p["planned"])
        # The prefetched rows stand for the tables as they are now if nothing has written the
        # cold table since the prefetch, or if the one write since then is the update of `after`,
        # whose rows were just read again.  Anything else leaves the state without a valid stamp
        # and the backward half reads the table.
        epoch0, version0 = p["stamp"]
        if after is None:
            valid = p["stamp"] == self._table_stamp()
        else:
            valid = (self._epoch == epoch0 + 1 and getattr(after[0], "update_epoch", None) == self._epoch
                     and self.cold_w._version == version0)
        self._stamp_forward(p["plan"], out, None if valid else (None, None))
        return out, (p["plan"], p["bufs"])

    def backward_keyed(self, state, grad, mode=ops.COMBINE_FAST, timing=None, fetched_rows="auto",
                       join=True, average=None):
        """Backward half: segmented sums of the cold class, whose update then starts on the cold
        stream while the hot class is summed and updated on the current stream; joins at the end.
        Returns (ukeys, sums, cnts, num_unique, class_split): the distinct rows in class order -
        cold ids ascending, then hot slots ascending with bit key_bits set.

        The cold update takes the old weights from the rows the forward half fetched for this
        batch instead of reading the cold table a second time (half the host-link traffic of the
        update) - but only while that is provably the same thing: `fetched_rows` = "auto" (the
        default) reuses them if this optimizer has issued no update on its tables since that
        forward half, torch's version counters of the cold table and of the rows are unchanged,
        and the optimizer was not constructed with reuse_fetched_rows=False; otherwise the table
        is read again.  Either way the result is the same bit for bit.  None always reads the
        table; a tensor is taken as the rows on the caller's word.

        `average`: None applies the per-id SUMS of the gradient rows (the combine of the
        benchmark configurations); "mean" divides every id's sum by its number of occurrences
        first, which is what the reference's update does with duplicate ids (unique_grads,
        python/EmbCache/sparse_optim.py:142-157,613); "one_plus" divides by one more than that
        (the reference's divisor when every row arrives with a count of one, :145-148).  The
        division happens inside the update kernels; the returned rows stay the sums and `cnts`
        the occurrences.

        join=False returns without making the current stream wait for the cold update; the caller
        then calls finish_prefetch(...) or join() before it reads the cold table on that stream."""
        plan, bufs = state
        cold = self._split_state()
        cur = torch.cuda.current_stream()
        n = plan.n
        fetched_rows = self._rows_to_reuse(plan, fetched_rows)
        plan.reused_rows = fetched_rows is not None
        self._epoch += 1
        plan.update_epoch = self._epoch
        out = (bufs["sums"][:n], bufs["cnts"][:n])
        if self.fuse_cold_sums:
            # the cold update sums the gradient rows of its runs itself (nearly every cold id
            # occurs once): it needs the plan and the gradients only, so it starts at once
            cold.wait_stream(cur)
            if cold != cur:
                grad.record_stream(cold)
        else:
            self._timed(timing, "cold_seg_sum", cur,
                        lambda: ops.combine_apply_class(plan, grad, 0, mode, out=out))
            cold_summed = torch.cuda.Event()
            cold_summed.record(cur)
            cold.wait_event(cold_summed)
        if fetched_rows is not None and cold != cur:
            fetched_rows.record_stream(cold)
        # beside a prefetch gather the link carries reads and writes at once, and a wide
        # write-only update then costs the gather more than it gains itself
        narrow = fetched_rows is not None and getattr(self, "_prefetching", False)
        if narrow:
            width = ops.set_host_link_blocks(ops.LINK_WRITE_ONLY, self.pipelined_update_blocks)
        with torch.cuda.stream(cold):
            self._timed(timing, "cold_update", cold,
                        lambda: self._update_keyed(plan, out[0], 0, fetched_rows,
                                                   grad_rows=grad if self.fuse_cold_sums else None,
                                                   out=out, average=average))
            self._cold_done = torch.cuda.Event()
            self._cold_done.record(cold)
        if narrow:
            ops.set_host_link_blocks(ops.LINK_WRITE_ONLY, width)
        self._timed(timing, "seg_sum", cur,
                    lambda: ops.combine_apply_class(plan, grad, 1, mode, out=out))
        if self.hot_ids.numel():
            self._timed(timing, "hot_update", cur,
                        lambda: self._update_keyed(plan, out[0], 1, out=out, average=average))
        if join:        # join=False: finish_prefetch (or join()) waits for the cold update later
            self.join()
        return plan.uids, out[0], out[1], plan.num_unique, plan.class_split

    def _update_keyed(self, plan, sums, which, fetched_rows=None, grad_rows=None, out=None,
                      average=None):
        raise NotImplementedError

    def distinct_ids_of(self, ukeys, num_unique, key_bits=None):
        """The real ids behind the class-ordered keys of a keyed step (one host synchronisation):
        cold keys are ids, hot keys name a slot of the hot set."""
        kb = key_bits if key_bits is not None else ops.key_bits_for(max(self.num_rows, self.hot_ids.numel(), 2))
        u = int(num_unique.item())
        if u < 0:
            raise ops._bound_error()
        k = ukeys[:u]
        hot = k >= (1 << kb)
        ids = k.clone()
        ids[hot] = self.hot_ids[k[hot] - (1 << kb)]
        return ids

    def step_split(self, idx, grad, mode=ops.COMBINE_FAST, plan=None, out=None, average=None):
        """step() on the split schedule; with `average` the returned rows are the averaged ones."""
        if plan is None:
            plan = ops.combine_plan(idx, self.dim, id_bound=self.num_rows, workspace=self._ws)
        else:
            torch.cuda.current_stream().wait_event(plan.ready)
        uids, sums, cnts, nu = ops.combine_apply(plan, grad, mode, out=out)
        self.update_split(uids, sums, nu, cnts=cnts, average=average)
        return uids, sums, cnts, nu

    def step(self, idx, grad, mode=ops.COMBINE_FAST, plan=None, out=None, average=None):
        """combine the per-occurrence gradients, then update every distinct row once.
        No host synchronisation.  `plan` = what prepare(idx) returned, if it was called.
        `average` = "mean" / "one_plus": the update divides every id's sum by its occurrences
        (plus one) inside its kernel; the returned rows stay the sums."""
        if plan is None:
            plan = ops.combine_plan(idx, self.dim, id_bound=self.num_rows, workspace=self._ws)
        else:
            torch.cuda.current_stream().wait_event(plan.ready)
        uids, sums, cnts, nu = ops.combine_apply(plan, grad, mode, out=out)
        self.update(uids, sums, nu, cnts=cnts, average=average)
        return uids, sums, cnts, nu


class SparseAdagrad(_SparseRowOptimizer):
    """s += g*g;  w -= lr * g / (sqrt(s) + eps) on the rows a step touches
    (torch.optim.Adagrad with lr_decay = weight_decay = initial_accumulator_value = 0)."""

    def __init__(self, weight_cold, hot_ids, lr=0.01, eps=1e-10, device="cuda",
                 state_on_device=False, cold_state=None, reuse_fetched_rows=True):
        """`cold_state` brings the cold Adagrad state instead of a new zero tensor; together with
        a row-strided `weight_cold` it allows one host table [N, 2, D] that holds the weight row
        and the state row of an id next to each other (weight_cold = t[:, 0], cold_state =
        t[:, 1]): one burst per cold row and direction over the host link.  Row-strided cold
        tables are served by the split schedule (fetch_split / update_split / step_split) and by
        the keyed one (forward_keyed / backward_keyed / prefetch_keyed); the one-kernel forms
        (fetch, update, step) need contiguous tables."""
        super().__init__(weight_cold, hot_ids, lr, device, state_on_device, reuse_fetched_rows)
        self.eps = eps
        if cold_state is not None:
            if tuple(cold_state.shape) != tuple(weight_cold.shape) or cold_state.dtype != torch.float32:
                raise RuntimeError("cold_state must be float32 of the weight table's shape")
            self.cold_s = cold_state
        else:
            self.cold_s = self._new_state_like(weight_cold)
        self.hot_s = torch.zeros_like(self.hot_w)

    def _update_class(self, index, grad, pos, count, hot):
        w, s = (self.hot_w, self.hot_s) if hot else (self.cold_w, self.cold_s)
        ops.adagrad_update_listed_(index, grad, pos, count, w, s, self.lr, self.eps)

    def _update_keyed(self, plan, sums, which, fetched_rows=None, grad_rows=None, out=None,
                      average=None):
        w, s = (self.hot_w, self.hot_s) if which else (self.cold_w, self.cold_s)
        ops.adagrad_update_class_(plan, sums, which, w, s, self.lr, self.eps, fetched_rows=fetched_rows,
                                  grad_rows=grad_rows, out=out if grad_rows is not None else None,
                                  average=average, cnts=out[1] if out is not None else None)

    def update(self, uids, grad, num_unique=None, cnts=None, average=None):
        self._epoch += 1
        ops.adagrad_update_(uids, grad, self.hot_w, self.hot_s, self.cold_w, self.cold_s,
                            self.hot_set, self.lr, self.eps, num_unique, cnts=cnts, average=average)


class SparseAdam(_SparseRowOptimizer):
    """The reference's SparseAdam.update (python/EmbCache/sparse_optim.py:590-685) as one kernel."""

    def __init__(self, weight_cold, hot_ids, lr=0.01, betas=(0.9, 0.999), eps=1e-8, device="cuda",
                 state_on_device=False, reuse_fetched_rows=True):
        super().__init__(weight_cold, hot_ids, lr, device, state_on_device, reuse_fetched_rows)
        self.betas, self.eps = betas, eps
        n, h = self.num_rows, self.hot_ids.numel()
        self.cold_step = self._new_state_like(weight_cold, (n,))
        self.cold_m = self._new_state_like(weight_cold)
        self.cold_v = self._new_state_like(weight_cold)
        self.hot_step = torch.zeros(h, dtype=torch.float32, device=self.device)
        self.hot_m = torch.zeros_like(self.hot_w)
        self.hot_v = torch.zeros_like(self.hot_w)

    def _tables(self, hot):
        return ((self.hot_w, self.hot_step, self.hot_m, self.hot_v) if hot else
                (self.cold_w, self.cold_step, self.cold_m, self.cold_v))

    def _update_class(self, index, grad, pos, count, hot):
        ops.adam_update_listed_(index, grad, pos, count, self._tables(hot), self.lr,
                                self.betas[0], self.betas[1], self.eps)

    def _update_keyed(self, plan, sums, which, fetched_rows=None, grad_rows=None, out=None,
                      average=None):
        ops.adam_update_class_(plan, sums, which, self._tables(bool(which)), self.lr,
                               self.betas[0], self.betas[1], self.eps, fetched_rows=fetched_rows,
                               grad_rows=grad_rows, out=out if grad_rows is not None else None,
                               average=average, cnts=out[1] if out is not None else None)

    def update(self, uids, grad, num_unique=None, cnts=None, average=None):
        self._epoch += 1
        ops.adam_update_(uids, grad, (self.hot_w, self.hot_step, self.hot_m, self.hot_v),
                         (self.cold_w, self.cold_step, self.cold_m, self.cold_v), self.hot_set,
                         self.lr, self.betas[0], self.betas[1], self.eps, num_unique,
                         cnts=cnts, average=average)

    def update_like_reference(self, idx, grad, cnt=None, is_unique=False, mode=ops.COMBINE_FAST):
        """The reference's SparseAdam.update(idx, grad, emb, cnt, is_unique)
        (python/EmbCache/sparse_optim.py:590-685) on this optimizer's table: duplicate ids get
        the MEAN of their gradient rows (unique_grads, :613; with `cnt` the divisor is one plus
        the summed counts, :145-148), already-unique input is divided by `cnt` if given (:607-611);
        then one Adam step on every distinct row.  Returns the distinct ids."""
        if is_unique:
            uids = idx
            vals = grad if cnt is None else grad / cnt.unsqueeze(1)
        else:
            uids, vals = unique_grads(idx, grad, cnt, id_bound=self.num_rows, mode=mode)
        self.update(uids, vals.contiguous())
        return uids
