"""Fused operators of the embedding-cache hot path over torch-ROCm tensors.

Thin, allocation-only wrappers around the C-ABI library: lookup against the sorted hot-ID set,
hot/cold split with stable compaction, cached_fetch / cached_set, combine and the sparse row
optimizers.  Every function launches on torch's current stream and returns without a host
synchronisation unless its name or docstring says otherwise; data-dependent sizes stay on the
device as one-element tensors (`num_unique`, `counts`) and outputs are padded to capacity.
"""
import ctypes

import torch

from . import _lib
from .EmbCacheLib import _check, _dev, _dev_or_pinned, _ptr, _stream

COMBINE_FAST = _lib.COMBINE_FAST
COMBINE_EXACT = _lib.COMBINE_EXACT

_NULL = ctypes.c_void_p(0)


def _i64(t, name):
    _check(t.dtype == torch.int64, "%s must be int64" % name)
    _dev(t, name)


def _opt(t):
    return _NULL if t is None else _ptr(t)


def _dcode(t):
    _check(t.dtype in (torch.float32, torch.float64), "Type can only be float or double")
    return _lib.F32 if t.dtype == torch.float32 else _lib.F64


class Workspace:
    """A reusable, 256-byte aligned device scratch buffer that grows on demand.  One workspace
    serves one stream at a time: work queued on another stream must be ordered after the work
    that used it before (the module's default workspaces are kept per stream for that reason)."""

    def __init__(self, device="cuda"):
        self.device = torch.device(device)
        self.buf = None

    def get(self, nbytes):
        if self.buf is None or self.buf.numel() < nbytes:
            # zero-filled: the cold-data cache's flush keeps a sticky status word at the start
            self.buf = torch.zeros(max(int(nbytes), 256), dtype=torch.uint8, device=self.device)
        else:
            # the caching allocator hands a freed block back to the stream it was allocated on:
            # tell it when the buffer is used on another one
            cur = torch.cuda.current_stream(self.device)
            if cur != getattr(self, "_stream", cur):
                self.buf.record_stream(cur)
        self._stream = torch.cuda.current_stream(self.device)
        return self.buf


_default_ws = {}


def _ws(device, kind):
    """The module's own workspace for (device, kind of operator, current stream): two streams
    never share scratch memory by default."""
    key = (str(device), kind, torch.cuda.current_stream(device).cuda_stream)
    if key not in _default_ws:
        _default_ws[key] = Workspace(device)
    return _default_ws[key]


def _bound_error():
    return RuntimeError("combine: an id lies outside [0, id_bound) (num_unique came back as -1); "
                        "pass id_bound=0 for ids without a known bound")


# ---- kernel timing -------------------------------------------------------------
KERNEL_CACHED_FETCH = _lib.KERNEL_CACHED_FETCH
KERNEL_SEG_SUM = _lib.KERNEL_SEG_SUM
KERNEL_ADAGRAD = _lib.KERNEL_ADAGRAD
KERNEL_RADIX_PASS = _lib.KERNEL_RADIX_PASS
KERNEL_HASH_ACCUMULATE = _lib.KERNEL_HASH_ACCUMULATE
KERNEL_ADAM = _lib.KERNEL_ADAM


def profile_kernel(kernel_id, start=None, stop=None):
    """Arms (or with kernel_id 0 disarms) a pair of torch.cuda.Event(enable_timing=True) that the
    library records around every later launch of that kernel, on the kernel's own stream.  The
    events must have been recorded once before, so that torch has created their handles."""
    if not kernel_id:
        _lib.call("hades_profile_kernel", 0, _NULL, _NULL)
        return
    _lib.call("hades_profile_kernel", int(kernel_id), ctypes.c_void_p(start.cuda_event),
              ctypes.c_void_p(stop.cuda_event))


LINK_COPY, LINK_READ_WRITE, LINK_WRITE_ONLY = 0, 1, 2


def set_host_link_blocks(use, blocks):
    """Width (workgroups) of the kernels whose table rows cross the host link: use = LINK_COPY
    (gather / scatter), LINK_READ_WRITE (update that reads and writes host rows) or
    LINK_WRITE_ONLY (update that only writes them); blocks = 0 restores the default.  Returns the
    width that was in force.  Process-wide; for tuning and measurement."""
    old = _lib.query("hades_get_host_link_blocks", int(use))
    _lib.call("hades_set_host_link_blocks", int(use), int(blocks))
    return old


def sort_config(one_sweep=None, spin_limit=None):
    """Chooses the sort under combine / bucketing / flush (process-wide): one_sweep True = one
    kernel per digit with bounded look-back waits, False = count + scatter kernels per digit;
    spin_limit = re-reads a tile spends on a predecessor that has published nothing before it
    recounts by itself (0: at once).  None leaves a setting alone.  Returns the form in force
    before the call (True = one sweep)."""
    old = bool(_lib.query("hades_sort_mode"))
    _lib.call("hades_sort_config", -1 if one_sweep is None else int(bool(one_sweep)),
              -1 if spin_limit is None else int(spin_limit))
    return old


def sort_wait_expiries(workspace):
    """Tiles of the last one-sweep sort in `workspace` (a Workspace, or the uint8 buffer itself)
    whose bounded wait ran out and which recounted instead.  One host synchronisation."""
    buf = workspace.buf if isinstance(workspace, Workspace) else workspace
    return int(buf[:4].view(torch.int32).item())


# ---- the hot set and lookup -----------------------------------------------------
class HotSet:
    """The ascending, duplicate-free hot ids on the device together with the bucket index that
    turns a lookup into one table read plus a search over a handful of ids.  Every operator that
    takes `sorted_hot` accepts either a plain int64 tensor (binary search) or a HotSet."""

    def __init__(self, sorted_hot, device=None, build_index=True):
        ids = torch.as_tensor(sorted_hot, dtype=torch.int64)
        if device is not None:
            ids = ids.to(device)
        _i64(ids, "sorted_hot")
        self.ids = ids
        self.index = None
        if build_index:
            nbytes = _lib.query("hades_hot_index_bytes", ids.numel())
            self.index = torch.empty(nbytes // 4, dtype=torch.int32, device=ids.device)
            _lib.call("hades_hot_index_build", _ptr(ids), ids.numel(), _ptr(self.index), nbytes,
                      _stream())

    def numel(self):
        return self.ids.numel()


def _hot_args(sorted_hot):
    """(ids pointer, count, index pointer) of a HotSet, a tensor or None."""
    if sorted_hot is None:
        return _NULL, 0, _NULL
    if isinstance(sorted_hot, HotSet):
        return _ptr(sorted_hot.ids), sorted_hot.ids.numel(), _opt(sorted_hot.index)
    _i64(sorted_hot, "sorted_hot")
    return _ptr(sorted_hot), sorted_hot.numel(), _NULL


def lookup(ids, sorted_hot, out=None):
    """loc[i] = slot of ids[i] in the ascending duplicate-free hot set, or -1."""
    _i64(ids, "ids")
    hp, hn, hi = _hot_args(sorted_hot)
    loc = out if out is not None else torch.empty_like(ids)
    _lib.call("hades_lookup_sorted", _ptr(ids), ids.numel(), hp, hn, hi, _ptr(loc), _stream())
    return loc


# ---- split + compaction -------------------------------------------------------
def split_padded(loc, workspace=None):
    """Hot/cold split of a looked-up batch, no host synchronisation.

    Returns (hot_mask bool[n], hot_pos int64[n], cold_pos int64[n], counts int64[2]); the first
    counts[0] entries of hot_pos and counts[1] of cold_pos are the ascending positions of each
    class, the rest is unspecified.
    """
    _i64(loc, "loc")
    n = loc.numel()
    hot_mask = torch.empty(n, dtype=torch.bool, device=loc.device)
    hot_pos = torch.empty(n, dtype=torch.int64, device=loc.device)
    cold_pos = torch.empty(n, dtype=torch.int64, device=loc.device)
    counts = torch.empty(2, dtype=torch.int64, device=loc.device)
    nbytes = _lib.query("hades_split_compact_workspace_bytes", n)
    ws = (workspace or _ws(loc.device, "split")).get(nbytes)
    _lib.call("hades_split_compact", _ptr(loc), n, _ptr(hot_mask), _ptr(hot_pos), _ptr(cold_pos),
              _ptr(counts), _ptr(ws), ws.numel(), _stream())
    return hot_mask, hot_pos, cold_pos, counts


def split(loc, workspace=None):
    """As split_padded, trimmed to size (one host synchronisation to read the two counts)."""
    hot_mask, hot_pos, cold_pos, counts = split_padded(loc, workspace)
    nh, nc = counts.tolist()
    return hot_mask, hot_pos[:nh], cold_pos[:nc]


def key_bits_for(num_rows):
    """Bits that hold every id of a table of num_rows rows (at least 1)."""
    return max(1, int(num_rows - 1).bit_length())


def lookup_split(ids, sorted_hot, num_live=None, workspace=None, out=None, sort_keys=None,
                 key_bits=0):
    """Lookup and hot/cold split in one call, no host synchronisation.

    Returns (loc int64[n], hot_pos int64[n], cold_pos int64[n], counts int64[2]): the slot of every
    id in the hot set (or -1), the ascending positions of the hot and of the cold ids (the first
    counts[0] / counts[1] entries are live) and the two counts.  `num_live` (int64[1] on the device)
    limits the batch to its first num_live[0] entries, e.g. the padded output of combine_padded.
    `out` may bring the four tensors.  `sort_keys` (int64[n]) receives the class-ordered sort key
    of every id - the id itself if cold, (1 << key_bits) | slot if hot - for combine_plan_classed."""
    _i64(ids, "ids")
    hp, hn, hi = _hot_args(sorted_hot)
    n, dev = ids.numel(), ids.device
    if out is None:
        out = (torch.empty(n, dtype=torch.int64, device=dev), torch.empty(n, dtype=torch.int64, device=dev),
               torch.empty(n, dtype=torch.int64, device=dev), torch.empty(2, dtype=torch.int64, device=dev))
    loc, hot_pos, cold_pos, counts = out
    _check(loc.numel() >= n and hot_pos.numel() >= n and cold_pos.numel() >= n and counts.numel() >= 2,
           "lookup_split outputs too small")
    nbytes = _lib.query("hades_split_compact_workspace_bytes", n)
    ws = (workspace or _ws(dev, "split")).get(nbytes)
    if sort_keys is not None:
        _i64(sort_keys, "sort_keys")
        _check(sort_keys.numel() >= n, "sort_keys too small")
    _lib.call("hades_lookup_split", _ptr(ids), _opt(num_live), n, hp, hn, hi, _ptr(loc), _NULL, _ptr(hot_pos),
              _ptr(cold_pos), _ptr(counts), _opt(sort_keys), int(key_bits), _ptr(ws), ws.numel(),
              _stream())
    return loc, hot_pos, cold_pos, counts


def _stride_of(table, dim):
    """Row stride in elements of a 2-D (or 1-D) table whose rows are contiguous."""
    if table.dim() == 1:
        _check(table.is_contiguous(), "1-D tables must be contiguous")
        return 1
    _check(table.stride(1) == 1 and table.stride(0) >= dim, "table rows must be contiguous")
    return table.stride(0)


def fetch_listed(table, index, pos_list, count, out, only_in=None, only_in_count=None):
    """out[p] = table[index[p]] for the first count[0] positions p of pos_list (device-side count:
    no host synchronisation).  `table` may be pinned host memory and may be a row-strided view.
    With `only_in` (ascending int64 ids) and `only_in_count` (int64[1] on the device) only the
    positions whose table row is among the first only_in_count[0] entries of only_in are fetched:
    the refresh of rows that were gathered ahead of an update of exactly those rows."""
    _i64(index, "index"); _i64(pos_list, "pos_list"); _i64(count, "count")
    _dev_or_pinned(table, "table", contiguous=False); _dev(out, "out")
    dim = 1 if out.dim() == 1 else out.size(1)
    _check(table.dtype == out.dtype, "table and out differ in dtype")
    if only_in is None:
        _lib.call("hades_fetch_listed", _ptr(table), _stride_of(table, dim), _ptr(index), _ptr(pos_list),
                  _ptr(count), pos_list.numel(), _ptr(out), dim, _dcode(out), _stream())
        return out
    _i64(only_in, "only_in"); _i64(only_in_count, "only_in_count")
    _lib.call("hades_fetch_listed_in_set", _ptr(table), _stride_of(table, dim), _ptr(index),
              _ptr(pos_list), _ptr(count), pos_list.numel(), _ptr(only_in), _ptr(only_in_count),
              only_in.numel(), _ptr(out), dim, _dcode(out), _stream())
    return out


def set_listed(src, table, index, pos_list, count):
    """table[index[p]] = src[p] for the first count[0] positions p of pos_list."""
    _i64(index, "index"); _i64(pos_list, "pos_list"); _i64(count, "count")
    _dev_or_pinned(table, "table", contiguous=False); _dev(src, "src")
    dim = 1 if src.dim() == 1 else src.size(1)
    _check(table.dtype == src.dtype, "table and src differ in dtype")
    _lib.call("hades_set_listed", _ptr(src), _ptr(table), _stride_of(table, dim), _ptr(index),
              _ptr(pos_list), _ptr(count), pos_list.numel(), dim, _dcode(src), _stream())


def adagrad_update_listed_(row_index, grad, pos_list, count, w, s, lr, eps, w_out=None):
    """Sparse Adagrad over the rows named by the first count[0] positions p of pos_list:
    g = grad[p]; r = row_index[p]; s[r] += g*g; w[r] -= lr * g / (sqrt(s[r]) + eps).  w and s are
    one table pair (device or pinned host) with the same row stride; they may be the two halves of
    one interleaved table.  `w_out` (float32 [positions, D] on the device) also receives the new
    weight row of every position."""
    _i64(row_index, "row_index"); _i64(pos_list, "pos_list"); _i64(count, "count"); _dev(grad, "grad")
    _check(grad.dtype == torch.float32 and grad.dim() == 2, "grad must be a 2-D float32 tensor")
    dim = grad.size(1)
    for name, t in (("w", w), ("s", s)):
        _dev_or_pinned(t, name, contiguous=False)
        _check(t.dtype == torch.float32 and t.dim() == 2 and t.size(1) == dim, "%s: wrong dtype/width" % name)
    stride = _stride_of(w, dim)
    _check(_stride_of(s, dim) == stride, "w and s must have the same row stride")
    if w_out is not None:
        _dev(w_out, "w_out")
        _check(w_out.dtype == torch.float32 and tuple(w_out.shape) == tuple(grad.shape),
               "w_out must be float32 of grad's shape")
    _lib.call("hades_adagrad_update_listed", _ptr(row_index), _ptr(grad), _ptr(pos_list), _ptr(count),
              pos_list.numel(), dim, _ptr(w), _ptr(s), stride, _opt(w_out), float(lr), float(eps),
              _stream())


def _adam_tables(tables, dim):
    """Checks one (w, step, mem, power) table set of the per-class Adam forms; returns the row stride."""
    w, step, m, v = tables
    for name, t in (("w", w), ("mem", m), ("power", v)):
        _dev_or_pinned(t, name, contiguous=False)
        _check(t.dtype == torch.float32 and t.dim() == 2 and t.size(1) == dim, "%s: wrong dtype/width" % name)
    _dev_or_pinned(step, "step")
    _check(step.dtype == torch.float32 and step.dim() == 1 and step.numel() == w.size(0),
           "step must be float32 with one entry per table row")
    stride = _stride_of(w, dim)
    _check(_stride_of(m, dim) == stride and _stride_of(v, dim) == stride,
           "w, mem and power must have the same row stride")
    return stride


def adam_update_listed_(row_index, grad, pos_list, count, tables, lr, beta1, beta2, eps):
    """SparseAdam (the arithmetic of adam_update_) over the rows named by the first count[0]
    positions p of pos_list: g = grad[p]; r = row_index[p]; one Adam step on row r of
    `tables` = (w, step, mem, power), one table set, device or pinned host."""
    _i64(row_index, "row_index"); _i64(pos_list, "pos_list"); _i64(count, "count"); _dev(grad, "grad")
    _check(grad.dtype == torch.float32 and grad.dim() == 2, "grad must be a 2-D float32 tensor")
    dim = grad.size(1)
    stride = _adam_tables(tables, dim)
    w, step, m, v = tables
    _lib.call("hades_adam_update_listed", _ptr(row_index), _ptr(grad), _ptr(pos_list), _ptr(count),
              pos_list.numel(), dim, _ptr(w), _ptr(step), _ptr(m), _ptr(v), stride, float(lr),
              float(beta1), float(beta2), float(eps), _stream())


def split3_padded(ids, class_table, workspace=None):
    """Three-way split by the int8 class table (0 local, 1 remote-hot, 2 remote-cold) with the
    compacted position lists; no host synchronisation.  Returns (masks[3], pos[3], counts[3])."""
    from .EmbCacheLib import _SPLIT_ITYPE
    _dev(ids, "ids"); _dev_or_pinned(class_table, "class_table")
    _check(class_table.dtype == torch.int8, "class_table must be int8")
    _check(ids.dtype in _SPLIT_ITYPE, "ids must be an integer tensor")
    n = ids.numel()
    masks = torch.empty((3, n), dtype=torch.bool, device=ids.device)
    pos = torch.empty((3, n), dtype=torch.int64, device=ids.device)
    counts = torch.empty(3, dtype=torch.int64, device=ids.device)
    nbytes = _lib.query("hades_split_compact_workspace_bytes", n)
    ws = (workspace or _ws(ids.device, "split")).get(nbytes)
    _lib.call("hades_split3_compact", _ptr(ids), _SPLIT_ITYPE[ids.dtype], _ptr(class_table), n,
              _ptr(masks[0]), _ptr(masks[1]), _ptr(masks[2]), _ptr(pos[0]), _ptr(pos[1]),
              _ptr(pos[2]), _ptr(counts), _ptr(ws), ws.numel(), _stream())
    return masks, pos, counts


# ---- cached_fetch / cached_set ------------------------------------------------
def _table_dim(*tables):
    ref = next(t for t in tables if t is not None)
    _check(ref.dim() in (1, 2), "tables must be 1-D or 2-D")
    for t in tables:
        if t is not None:
            _check(t.dim() == ref.dim() and t.dtype == ref.dtype, "table shape/dtype mismatch")
            _check(ref.dim() == 1 or t.size(1) == ref.size(1), "row widths differ")
    return 1 if ref.dim() == 1 else ref.size(1)


def cached_fetch(cold, hot, ids, sorted_hot, out=None, return_loc=False):
    """out[i] = hot[slot] if ids[i] is in sorted_hot (slot = its rank there) else cold[ids[i]].

    `cold` may be a device tensor or a pinned host tensor (read zero-copy).  The lookup runs
    inside the gather kernel."""
    _i64(ids, "ids")
    hp, hn, hi = _hot_args(sorted_hot)
    _dev_or_pinned(cold, "cold"); _dev(hot, "hot")
    dim = _table_dim(cold, hot)
    n = ids.numel()
    shape = (n,) if hot.dim() == 1 else (n, dim)
    if out is None:
        out = torch.empty(shape, dtype=hot.dtype, device=ids.device)
    else:
        _dev(out, "out")
        _check(tuple(out.shape) == shape and out.dtype == hot.dtype, "out has the wrong shape/dtype")
    loc = torch.empty_like(ids) if return_loc else None
    _lib.call("hades_cached_fetch", _ptr(cold), _ptr(hot), _ptr(ids), n, hp, hn, hi, _ptr(out),
              _opt(loc), dim, _dcode(hot), _stream())
    return (out, loc) if return_loc else out


def cached_fetch_loc(cold, hot, ids, loc, out=None):
    """cached_fetch when the slots are already known (loc from `lookup`)."""
    _i64(ids, "ids"); _i64(loc, "loc")
    _dev_or_pinned(cold, "cold"); _dev(hot, "hot")
    _check(loc.numel() == ids.numel(), "loc and ids differ in length")
    dim = _table_dim(cold, hot)
    n = ids.numel()
    shape = (n,) if hot.dim() == 1 else (n, dim)
    if out is None:
        out = torch.empty(shape, dtype=hot.dtype, device=ids.device)
    _lib.call("hades_cached_fetch_loc", _ptr(cold), _ptr(hot), _ptr(ids), _ptr(loc), n, _ptr(out),
              dim, _dcode(hot), _stream())
    return out


def cached_set(src, cold, hot, ids, sorted_hot):
    """(hot[slot] if ids[i] in sorted_hot else cold[ids[i]]) = src[i]; ids must be duplicate-free
    for a defined result."""
    _i64(ids, "ids")
    hp, hn, hi = _hot_args(sorted_hot)
    _dev(src, "src"); _dev_or_pinned(cold, "cold"); _dev(hot, "hot")
    dim = _table_dim(cold, hot, src)
    _check(src.size(0) >= ids.numel(), "src has fewer rows than ids has entries")
    _lib.call("hades_cached_set", _ptr(src), _ptr(cold), _ptr(hot), _ptr(ids), ids.numel(),
              hp, hn, hi, dim, _dcode(hot), _stream())


# ---- combine ------------------------------------------------------------------
def combine_padded(idx, grad, id_bound=0, mode=COMBINE_FAST, return_inverse=False, workspace=None,
                   out=None):
    """Sort + dedup + segment-sum, no host synchronisation.

    Returns (uids int64[n], sums float32[n, D], cnts int64[n], num_unique int64[1]) - and
    inverse int32[n] when asked - of which the first num_unique[0] rows are live.
    id_bound > 0 promises 0 <= idx < id_bound and shortens the sort.
    """
    _i64(idx, "idx"); _dev(grad, "grad")
    _check(grad.dtype == torch.float32 and grad.dim() == 2, "grad must be a 2-D float32 tensor")
    n, dim = idx.numel(), grad.size(1)
    _check(grad.size(0) == n, "grad must have one row per id")
    dev = idx.device
    if out is None:
        uids = torch.empty(n, dtype=torch.int64, device=dev)
        sums = torch.empty((n, dim), dtype=torch.float32, device=dev)
        cnts = torch.empty(n, dtype=torch.int64, device=dev)
        num_unique = torch.empty(1, dtype=torch.int64, device=dev)
    else:
        uids, sums, cnts, num_unique = out
    inverse = torch.empty(n, dtype=torch.int32, device=dev) if return_inverse else None
    nbytes = _lib.query("hades_combine_workspace_bytes", n, dim)
    ws = (workspace or _ws(dev, "combine")).get(nbytes)
    _lib.call("hades_combine", _ptr(idx), _ptr(grad), n, dim, int(id_bound), int(mode), _ptr(uids),
              _ptr(sums), _ptr(cnts), _ptr(num_unique), _opt(inverse), _ptr(ws), ws.numel(),
              _stream())
    if return_inverse:
        return uids, sums, cnts, num_unique, inverse
    return uids, sums, cnts, num_unique


class CombinePlan:
    """The id-only half of a combine: sort permutation and run boundaries (kept in `workspace`),
    the distinct ids and their number.  Made by combine_plan, consumed by combine_apply."""

    def __init__(self, n, dim, id_bound, uids, num_unique, inverse, workspace, buf):
        self.n, self.dim, self.id_bound = n, dim, id_bound
        self.uids, self.num_unique, self.inverse = uids, num_unique, inverse
        self.workspace = workspace
        # the buffer the plan was written into: a workspace that grew or was given to a later
        # plan no longer holds it
        self._buf_ptr, self._buf_len = buf.data_ptr(), buf.numel()
        workspace._plan = self

    def check_live(self):
        buf = self.workspace.buf
        if (buf is None or buf.data_ptr() != self._buf_ptr or buf.numel() != self._buf_len
                or getattr(self.workspace, "_plan", None) is not self):
            raise RuntimeError("combine plan invalidated: its workspace was reallocated or reused "
                               "by a later plan before combine_apply consumed it")
        return buf


def combine_plan(idx, dim, id_bound=0, return_inverse=False, workspace=None, out=None):
    """Sorts the ids and finds the runs; needs no gradients, so it can run as soon as the ids of a
    batch are known (e.g. at forward time, on another stream).  `workspace` is a Workspace that must
    not be used by anything else until combine_apply has consumed the plan.  `out` = (uids int64[n],
    num_unique int64[1]) to write into preallocated tensors."""
    _i64(idx, "idx")
    n, dev = idx.numel(), idx.device
    if out is None:
        uids = torch.empty(n, dtype=torch.int64, device=dev)
        num_unique = torch.empty(1, dtype=torch.int64, device=dev)
    else:
        uids, num_unique = out
    inverse = torch.empty(n, dtype=torch.int32, device=dev) if return_inverse else None
    workspace = workspace or Workspace(dev)
    ws = workspace.get(_lib.query("hades_combine_workspace_bytes", n, int(dim)))
    _lib.call("hades_combine_plan", _ptr(idx), n, int(dim), int(id_bound), _ptr(uids),
              _ptr(num_unique), _opt(inverse), _ptr(ws), ws.numel(), _stream())
    return CombinePlan(n, int(dim), int(id_bound), uids, num_unique, inverse, workspace, ws)


def combine_apply(plan, grad, mode=COMBINE_FAST, out=None):
    """Segmented row sums of `grad` under a plan.  Returns (uids, sums, cnts, num_unique) like
    combine_padded; `out` = (sums float32[n, D], cnts int64[n]) to write into preallocated tensors."""
    _dev(grad, "grad")
    _check(grad.dtype == torch.float32 and grad.dim() == 2, "grad must be a 2-D float32 tensor")
    _check(grad.size(0) == plan.n and grad.size(1) == plan.dim, "grad does not match the plan")
    dev = grad.device
    if out is None:
        sums = torch.empty((plan.n, plan.dim), dtype=torch.float32, device=dev)
        cnts = torch.empty(plan.n, dtype=torch.int64, device=dev)
    else:
        sums, cnts = out
    ws = plan.check_live()
    _lib.call("hades_combine_apply", _ptr(grad), plan.n, plan.dim, plan.id_bound, int(mode),
              _ptr(sums), _ptr(cnts), _ptr(plan.num_unique), _ptr(ws), ws.numel(), _stream())
    return plan.uids, sums, cnts, plan.num_unique


def combine_plan_classed(keys, dim, key_bits, workspace=None, out=None, first_pos=None):
    """combine_plan over the class-ordered keys that lookup_split(..., sort_keys=, key_bits=) made.
    The plan also carries class_split (int64[2] on the device): first sorted position and first
    run of the hot class.  `out` = (ukeys int64[n], num_unique int64[1], class_split int64[2]).
    `first_pos` (int32[n]) receives the batch position of the first occurrence of every distinct
    key (plan.first_pos)."""
    _i64(keys, "keys")
    n, dev = keys.numel(), keys.device
    if out is None:
        out = (torch.empty(n, dtype=torch.int64, device=dev), torch.empty(1, dtype=torch.int64, device=dev),
               torch.empty(2, dtype=torch.int64, device=dev))
    ukeys, num_unique, class_split = out
    workspace = workspace or Workspace(dev)
    ws = workspace.get(_lib.query("hades_combine_workspace_bytes", n, int(dim)))
    bound, thr = 1 << (int(key_bits) + 1), 1 << int(key_bits)
    if first_pos is not None:
        _check(first_pos.dtype == torch.int32 and first_pos.is_cuda and first_pos.numel() >= n,
               "first_pos must be an int32 device tensor of n entries")
    _lib.call("hades_combine_plan_classed", _ptr(keys), n, int(dim), bound, thr, _ptr(ukeys),
              _ptr(num_unique), _ptr(class_split), _opt(first_pos), _ptr(ws), ws.numel(), _stream())
    plan = CombinePlan(n, int(dim), bound, ukeys, num_unique, None, workspace, ws)
    plan.class_split, plan.key_bits, plan.first_pos = class_split, int(key_bits), first_pos
    return plan


def combine_apply_class(plan, grad, which, mode=COMBINE_FAST, out=None):
    """Segmented sums and counts of one class of a classed plan: which = 0 the cold runs (rows
    [0, class_split[1]) of the outputs), 1 the hot runs (the rows after them).  Both calls write
    into the same `out` = (sums float32[n, D], cnts int64[n])."""
    _dev(grad, "grad")
    _check(grad.dtype == torch.float32 and grad.dim() == 2, "grad must be a 2-D float32 tensor")
    _check(grad.size(0) == plan.n and grad.size(1) == plan.dim, "grad does not match the plan")
    if out is None:
        out = (torch.empty((plan.n, plan.dim), dtype=torch.float32, device=grad.device),
               torch.empty(plan.n, dtype=torch.int64, device=grad.device))
    sums, cnts = out
    ws = plan.check_live()
    _lib.call("hades_combine_apply_class", _ptr(grad), plan.n, plan.dim, plan.id_bound, int(mode),
              int(which), _ptr(sums), _ptr(cnts), _ptr(plan.num_unique), _ptr(plan.class_split),
              _ptr(ws), ws.numel(), _stream())
    return sums, cnts


def _class_rows(plan, dim, fetched_rows):
    """first_pos tensor to pass with `fetched_rows` (or None), after checking both"""
    if fetched_rows is None:
        return None
    _dev(fetched_rows, "fetched_rows")
    _check(plan.first_pos is not None, "the plan was made without first_pos")
    _check(fetched_rows.dtype == torch.float32 and tuple(fetched_rows.shape) == (plan.n, dim),
           "fetched_rows must be float32 [n, dim]")
    return plan.first_pos


def _summing_outputs(plan, grad_rows, out):
    """Checks the per-query gradient rows and the optional (sums, cnts) outputs of a summing
    class update; returns (sums or None, cnts or None, the plan's live workspace buffer)."""
    _dev(grad_rows, "grad_rows")
    _check(grad_rows.dtype == torch.float32 and tuple(grad_rows.shape) == (plan.n, plan.dim),
           "grad_rows must be float32 [n, dim]: one gradient row per query of the planned batch")
    sums = cnts = None
    if out is not None:
        sums, cnts = out
        _dev(sums, "sums"); _i64(cnts, "cnts")
        _check(sums.dtype == torch.float32 and sums.size(0) >= plan.n and sums.size(1) == plan.dim
               and cnts.numel() >= plan.n, "summing outputs must be float32 [n, dim] and int64 [n]")
    return sums, cnts, plan.check_live()


AVERAGE = {None: 0, "sum": 0, "mean": 1, "one_plus": 2}


def _average_code(average):
    _check(average in AVERAGE, "average must be None, 'mean' or 'one_plus'")
    return AVERAGE[average]


def adagrad_update_class_(plan, sums, which, w, s, lr, eps, fetched_rows=None, grad_rows=None,
                          out=None, average=None, cnts=None):
    """Sparse Adagrad over one class of a classed plan: the table row of run u is
    plan.uids[u] & (2^key_bits - 1) - the id for the cold class, the slot for the hot class.
    `fetched_rows` (float32[n, D], the rows the forward pass fetched for this batch) makes the
    kernel take the old weight rows from there (row plan.first_pos[u]) instead of reading the
    table again; valid only while nothing has written those table rows since the fetch.
    With `grad_rows` (float32[n, D], one gradient row per query; `sums` is then ignored and may be
    None) the kernel sums the rows of every run itself, in occurrence order from +0.0 - the
    deterministic-order sum - instead of reading them from `sums`; `out` = (sums, cnts) then
    receives the summed rows and counts of the class.
    `average` = "mean" divides every row by its number of occurrences before the update
    (unique_grads, python/EmbCache/sparse_optim.py:150-156), "one_plus" by one more (:145-148);
    without grad_rows the occurrences come from `cnts` (the counts combine_apply_class wrote)."""
    avg = _average_code(average)
    if avg and grad_rows is None:
        _check(cnts is not None, "averaging needs cnts")
        _i64(cnts, "cnts")
    dim = plan.dim if grad_rows is not None else sums.size(1)
    for name, t in (("w", w), ("s", s)):
        _dev_or_pinned(t, name, contiguous=False)
        _check(t.dtype == torch.float32 and t.dim() == 2 and t.size(1) == dim, "%s: wrong dtype/width" % name)
    stride = _stride_of(w, dim)
    _check(_stride_of(s, dim) == stride, "w and s must have the same row stride")
    fp = _class_rows(plan, dim, fetched_rows)
    if grad_rows is not None:
        so, co, ws = _summing_outputs(plan, grad_rows, out)
        _lib.call("hades_adagrad_update_class_summing", _ptr(plan.uids), _ptr(grad_rows), plan.n,
                  plan.id_bound, _ptr(plan.num_unique), _ptr(plan.class_split), int(which),
                  (1 << plan.key_bits) - 1, dim, _ptr(w), _ptr(s), stride, _opt(fetched_rows), _opt(fp),
                  _opt(so), _opt(co), avg, float(lr), float(eps), _ptr(ws), ws.numel(), _stream())
        return
    _dev(sums, "sums")
    _lib.call("hades_adagrad_update_class", _ptr(plan.uids), _ptr(sums), _ptr(plan.num_unique),
              _ptr(plan.class_split), int(which), (1 << plan.key_bits) - 1, plan.uids.numel(), dim,
              _ptr(w), _ptr(s), stride, _opt(fetched_rows), _opt(fp), _opt(cnts if avg else None), avg,
              float(lr), float(eps), _stream())


def adam_update_class_(plan, sums, which, tables, lr, beta1, beta2, eps, fetched_rows=None,
                       grad_rows=None, out=None, average=None, cnts=None):
    """SparseAdam over one class of a classed plan; rows, `fetched_rows`, `grad_rows`, `out`,
    `average` and `cnts` as in adagrad_update_class_, `tables` = (w, step, mem, power) of that
    class."""
    avg = _average_code(average)
    if avg and grad_rows is None:
        _check(cnts is not None, "averaging needs cnts")
        _i64(cnts, "cnts")
    dim = plan.dim if grad_rows is not None else sums.size(1)
    stride = _adam_tables(tables, dim)
    w, step, m, v = tables
    fp = _class_rows(plan, dim, fetched_rows)
    if grad_rows is not None:
        so, co, ws = _summing_outputs(plan, grad_rows, out)
        _lib.call("hades_adam_update_class_summing", _ptr(plan.uids), _ptr(grad_rows), plan.n,
                  plan.id_bound, _ptr(plan.num_unique), _ptr(plan.class_split), int(which),
                  (1 << plan.key_bits) - 1, dim, _ptr(w), _ptr(step), _ptr(m), _ptr(v), stride,
                  _opt(fetched_rows), _opt(fp), _opt(so), _opt(co), avg, float(lr), float(beta1),
                  float(beta2), float(eps), _ptr(ws), ws.numel(), _stream())
        return
    _dev(sums, "sums")
    _lib.call("hades_adam_update_class", _ptr(plan.uids), _ptr(sums), _ptr(plan.num_unique),
              _ptr(plan.class_split), int(which), (1 << plan.key_bits) - 1, plan.uids.numel(), dim,
              _ptr(w), _ptr(step), _ptr(m), _ptr(v), stride, _opt(fetched_rows), _opt(fp),
              _opt(cnts if avg else None), avg, float(lr), float(beta1), float(beta2), float(eps),
              _stream())


def combine(idx, grad, id_bound=0, mode=COMBINE_FAST, workspace=None):
    """As combine_padded, trimmed to the number of distinct ids (one host synchronisation).
    Raises if an id violated id_bound."""
    uids, sums, cnts, num_unique = combine_padded(idx, grad, id_bound, mode, workspace=workspace)
    u = int(num_unique.item())
    if u < 0:
        raise _bound_error()
    return uids[:u], sums[:u], cnts[:u]


def combine_static(idx, grad, id_bound=0, mode=COMBINE_FAST, out=None):
    """combine_padded on the library's own fixed scratch array (no workspace, nothing allocated by
    the library): for callers that cannot allocate.  Batches whose scratch need exceeds
    COMBINE_STATIC_SCRATCH_BYTES are refused.  Calls that overlap on one GPU race on the array."""
    _i64(idx, "idx"); _dev(grad, "grad")
    _check(grad.dtype == torch.float32 and grad.dim() == 2, "grad must be a 2-D float32 tensor")
    n, dim = idx.numel(), grad.size(1)
    _check(grad.size(0) == n, "grad must have one row per id")
    dev = idx.device
    if out is None:
        out = (torch.empty(n, dtype=torch.int64, device=dev),
               torch.empty((n, dim), dtype=torch.float32, device=dev),
               torch.empty(n, dtype=torch.int64, device=dev),
               torch.empty(1, dtype=torch.int64, device=dev))
    uids, sums, cnts, num_unique = out
    _lib.call("hades_combine_static", _ptr(idx), _ptr(grad), n, dim, int(id_bound), int(mode),
              _ptr(uids), _ptr(sums), _ptr(cnts), _ptr(num_unique), _NULL, _stream())
    return uids, sums, cnts, num_unique


def rows_div_count_(sums, cnts, num_unique=None, one_plus=False):
    """In place: sums[u] /= (cnts[u] + one_plus) for the live rows."""
    _dev(sums, "sums"); _i64(cnts, "cnts")
    _lib.call("hades_rows_div_count", _ptr(sums), _ptr(cnts), _opt(num_unique), sums.size(0),
              sums.size(1), 1 if one_plus else 0, _stream())
    return sums


# ---- row optimizers -----------------------------------------------------------
def adagrad_update_(uids, grad, hot_w, hot_s, cold_w, cold_s, sorted_hot, lr, eps,
                    num_unique=None, cnts=None, average=None):
    """Sparse Adagrad over the rows named by the duplicate-free `uids`, in place:
    s += g*g;  w -= lr * g / (sqrt(s) + eps), each row in the hot tables if its id is in
    sorted_hot, else in the cold tables (device or pinned host).  `average` = "mean" / "one_plus"
    with `cnts` (the combine's counts) divides every row by its count (plus one) first."""
    avg = _average_code(average)
    if avg:
        _check(cnts is not None, "averaging needs cnts")
        _i64(cnts, "cnts")
    _i64(uids, "uids"); _dev(grad, "grad")
    _check(grad.dtype == torch.float32 and grad.dim() == 2, "grad must be a 2-D float32 tensor")
    dim = grad.size(1)
    hp, hn, hi = _hot_args(sorted_hot)
    for name, t in (("hot_w", hot_w), ("hot_s", hot_s)):
        if t is not None:
            _dev(t, name)
            _check(t.dtype == torch.float32 and t.size(1) == dim, "%s: wrong dtype/width" % name)
    for name, t in (("cold_w", cold_w), ("cold_s", cold_s)):
        if t is not None:
            _dev_or_pinned(t, name)
            _check(t.dtype == torch.float32 and t.size(1) == dim, "%s: wrong dtype/width" % name)
    _check(grad.size(0) >= uids.numel(), "grad has fewer rows than uids has entries")
    _lib.call("hades_adagrad_update", _ptr(uids), _ptr(grad), _opt(num_unique), uids.numel(), dim,
              hp, hn, hi, _opt(hot_w), _opt(hot_s), _opt(cold_w), _opt(cold_s),
              _opt(cnts if avg else None), avg, float(lr), float(eps), _stream())


def adam_update_(uids, grad, hot, cold, sorted_hot, lr, beta1, beta2, eps, num_unique=None,
                 cnts=None, average=None):
    """SparseAdam row update in place.  `hot` and `cold` are (w, step, mem, power) tuples;
    `cnts` / `average` as in adagrad_update_."""
    avg = _average_code(average)
    if avg:
        _check(cnts is not None, "averaging needs cnts")
        _i64(cnts, "cnts")
    _i64(uids, "uids"); _dev(grad, "grad")
    dim = grad.size(1)
    hp, hn, hi = _hot_args(sorted_hot)
    hot = hot if hot is not None else (None, None, None, None)
    _lib.call("hades_adam_update", _ptr(uids), _ptr(grad), _opt(num_unique), uids.numel(), dim,
              hp, hn, hi, _opt(hot[0]), _opt(hot[1]), _opt(hot[2]), _opt(hot[3]),
              _opt(cold[0]), _opt(cold[1]), _opt(cold[2]), _opt(cold[3]), _opt(cnts if avg else None), avg,
              float(lr), float(beta1), float(beta2), float(eps), _stream())


# ---- cold-gradient accumulator ------------------------------------------------
class ColdGradAccumulator:
    """Open-addressing hash table in HBM: int64 id -> float32[dim] running sum and a count.

    accumulate() adds a duplicate-free batch (combine it first); flush() returns every live entry
    in ascending id order and empties the table.  The arithmetic is that of the reference's cache
    server (python/EmbCache/server.py:546-562, 346-497) with a flush decided by the caller.
    """

    def __init__(self, num_slots, dim, id_bound=0, device="cuda"):
        _check(num_slots > 0 and (num_slots & (num_slots - 1)) == 0, "num_slots must be a power of two")
        self.num_slots, self.dim, self.id_bound = int(num_slots), int(dim), int(id_bound)
        self.device = torch.device(device)
        # key and count of a slot share one 16-byte record: a probe and the count update touch one
        # memory sector instead of two
        self.slots = torch.empty((num_slots, 2), dtype=torch.int64, device=self.device)
        self.keys, self.cnt = self.slots[:, 0], self.slots[:, 1]
        self.accum = torch.empty((num_slots, dim), dtype=torch.float32, device=self.device)
        self.status = torch.zeros(1, dtype=torch.int32, device=self.device)
        self._ws = Workspace(self.device)
        self.clear()

    def clear(self):
        _lib.call("hades_hash_clear", _ptr(self.keys), _ptr(self.accum), _ptr(self.cnt),
                  self.num_slots, self.dim, 2, _stream())

    def accumulate(self, ids, grad, cnt=None, num_rows=None):
        _i64(ids, "ids"); _dev(grad, "grad")
        _check(grad.dtype == torch.float32 and grad.dim() == 2 and grad.size(1) == self.dim,
               "grad must be float32 [rows, dim]")
        _lib.call("hades_hash_accumulate", _ptr(self.keys), _ptr(self.accum), _ptr(self.cnt),
                  self.num_slots, _ptr(ids), _ptr(grad), _opt(cnt), _opt(num_rows), ids.numel(),
                  self.dim, _ptr(self.status), 2, _stream())

    def flush_padded(self, cap, out=None):
        """Returns (ids int64[cap], sums float32[cap, dim], cnts int64[cap], num_out int64[1]);
        `out` may bring these four tensors to avoid their allocation."""
        dev = self.device
        if out is not None:
            out_ids, out_sums, out_cnts, num_out = out
            _check(out_ids.numel() >= cap and out_sums.size(0) >= cap and out_cnts.numel() >= cap,
                   "flush outputs smaller than cap")
        else:
            out_ids = torch.empty(cap, dtype=torch.int64, device=dev)
            out_sums = torch.empty((cap, self.dim), dtype=torch.float32, device=dev)
            out_cnts = torch.empty(cap, dtype=torch.int64, device=dev)
            num_out = torch.empty(1, dtype=torch.int64, device=dev)
        nbytes = _lib.query("hades_hash_flush_workspace_bytes", self.num_slots, cap)
        ws = self._ws.get(nbytes)
        _lib.call("hades_hash_flush", _ptr(self.keys), _ptr(self.accum), _ptr(self.cnt),
                  self.num_slots, self.dim, self.id_bound, _ptr(out_ids), _ptr(out_sums),
                  _ptr(out_cnts), _ptr(num_out), cap, _ptr(self.status), 2, _ptr(ws), ws.numel(),
                  _stream())
        return out_ids, out_sums, out_cnts, num_out

    def flush(self, cap=None):
        """Trimmed flush (one host synchronisation).  Raises if the table overflowed."""
        cap = cap or self.num_slots
        ids, sums, cnts, num_out = self.flush_padded(cap)
        n = int(num_out.item())
        st = int(self.status.item())
        if st:
            self.status.zero_()
            raise RuntimeError("cold-gradient accumulator overflow (status %d): table full or "
                               "flush capacity too small" % st)
        return ids[:n], sums[:n], cnts[:n]


# ---- pre-exchange bucketing ------------------------------------------------------
def bucket_by_owner(ids, grad=None, cnt=None, partition_range=None, local_num_gpus=1,
                    num_owners=None, return_perm=False, workspace=None):
    """Groups a batch by the rank that owns each id, as swap_gradients does before its all-to-all
    (python/EmbCache/sparse_optim.py:33-50), without a host synchronisation.

    owner = id % local_num_gpus, plus (index of the id's range in partition_range) * local_num_gpus
    when a partition range is given.  Returns (ids_out, grad_out, cnt_out, split_sizes[, perm]):
    the inputs stably sorted by owner (None where the input was None), split_sizes int64[num_owners]
    on the device, and perm int64[n] (input position of every output row) when asked.
    """
    _i64(ids, "ids")
    n = ids.numel()
    dev = ids.device
    if partition_range is not None:
        _i64(partition_range, "partition_range")
        num_part = partition_range.numel()
        _check(num_part >= 1, "partition_range must not be empty")
    else:
        num_part = 0
    if num_owners is None:
        num_owners = max(1, num_part) * int(local_num_gpus)
    dim, dcode = 1, _lib.F32
    grad_out = cnt_out = perm = None
    if grad is not None:
        _dev(grad, "grad")
        _check(grad.dim() == 2 and grad.size(0) == n, "grad must be [len(ids), dim]")
        dim, dcode = grad.size(1), _dcode(grad)
        grad_out = torch.empty_like(grad)
    if cnt is not None:
        _i64(cnt, "cnt")
        _check(cnt.numel() == n, "cnt must have one entry per id")
        cnt_out = torch.empty_like(cnt)
    if return_perm:
        perm = torch.empty(n, dtype=torch.int64, device=dev)
    ids_out = torch.empty_like(ids)
    split_sizes = torch.empty(int(num_owners), dtype=torch.int64, device=dev)
    nbytes = _lib.query("hades_bucket_workspace_bytes", n)
    ws = (workspace or _ws(dev, "bucket")).get(nbytes)
    _lib.call("hades_bucket_by_owner", _ptr(ids), n, _opt(partition_range), num_part,
              int(local_num_gpus), int(num_owners), _opt(grad), dim, dcode, _opt(cnt),
              _ptr(ids_out), _opt(grad_out), _opt(cnt_out), _ptr(split_sizes), _opt(perm),
              _ptr(ws), ws.numel(), _stream())
    if return_perm:
        return ids_out, grad_out, cnt_out, split_sizes, perm
    return ids_out, grad_out, cnt_out, split_sizes
