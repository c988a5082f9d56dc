"""CPU restatement of the HADES embedding-cache hot path.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may import it.  Nothing under hades_amd/ imports it and nothing here
touches a GPU.

Every function restates one reference function and cites it.  Native (CUDA) functions of the
reference are restated with numpy; the Python functions of the reference (only_unique_grads,
unique_grads, SparseAdam.update) are restated with the same torch CPU calls the reference makes,
next to an independent numpy restatement used to cross-check them.

How each function is pinned (tests/test_oracle.py):
  upper_bound / owner_rank / reminder : Python bisect and C remainder on random and edge inputs;
                                        the split-size recipe of test/test_binarysearch2.py:13-27
  lookup_sorted                       : brute-force membership on small inputs, edge cases
  split_masks / split_compact         : the CPU split of test/test_split.py:30-37, mask invariants
  fetch* / set*                       : the recipes of test/test_cached_fetch.py:22,43,
                                        test/test_cached_set.py:22,26, test/test_fetch.py:16,
                                        test/test_combine.py:16 (plain torch indexing, bit-exact),
                                        independence from which rows are cached
  combine                             : torch.unique + index_add_ (the reference's own calls) vs
                                        the numpy stable-sort restatement vs float64 sums; closed
                                        forms (all ids distinct, all ids equal), sum(cnt) == n
  adagrad                             : torch.optim.Adagrad on the gathered rows; g == 0 leaves w
                                        unchanged; first-step closed form
  adam                                : PARTLY PINNED.  Closed forms: from zero state, and again with
                                        the same gradient, every step is -lr * sign(g), m and v
                                        follow (1 - beta^t) g and (1 - beta^t) g^2; g = 0 moves
                                        nothing.  torch.optim.Adam (same mathematics) agrees to
                                        2e-4 of one update on w and to rounding on m and v; the
                                        reference forms 1 - beta^t in float32
                                        (python/EmbCache/sparse_optim.py:652-655), a 6e-5 relative
                                        error no library routine reproduces, and holds no test or
                                        vector for it: below that level the weight update is
                                        parity unpinned
  hash accumulator                    : a Python dict model; flush(accumulate(batches)) equals
                                        combine(concat(batches))
  hot placement                       : the reference's own argsort recipe, cache.py:165-171
  bucket_by_owner                     : torch.sort(stable=True) + bincount over the reference's
                                        owner formula; brute-force bucket membership in input order
  SACacheIndexModel                   : a sequence worked by hand from src/cache/cache_line.h, and
                                        the reference's own cache_line class compiled into
                                        oracle/_ref (ref_sacache_driver.cpp) on random sequences
  ColdCacheServerModel                : per-id bookkeeping (pending sum, count, iteration counter,
                                        threshold) without evictions; a worked case for the dense
                                        local part
The C restatement of the native functions (hades_oracle.c) is checked against this module; the
committed vectors of tests/golden/ (made without this module) are checked in tests/test_golden.py.
"""
import numpy as np
import torch


# ---------------------------------------------------------------------------
# routing arithmetic: src/cuda/binary_search.cu
# ---------------------------------------------------------------------------
def upper_bound(sorted_range, values):
    """cub::UpperBound as used by BinarySearchKernel2 (src/cuda/binary_search.cu:24-33):
    number of entries of the ascending range that are <= value.  Output dtype = input dtype (:64)."""
    sorted_range = np.asarray(sorted_range)
    values = np.asarray(values)
    return np.searchsorted(sorted_range, values, side="right").astype(values.dtype)


def c_remainder(values, m):
    """C `%` (sign follows the dividend), what ReminderKernel computes (src/cuda/binary_search.cu:36-43)."""
    values = np.asarray(values)
    return np.fmod(values, values.dtype.type(m)).astype(values.dtype)


def owner_rank(values, range_partition, local_num_gpus):
    """BinarySearchKernel (src/cuda/binary_search.cu:11-21):
    (UpperBound(range_partition, v) - 1) * local_num_gpus + v % local_num_gpus."""
    values = np.asarray(values)
    rank = np.searchsorted(np.asarray(range_partition), values, side="right").astype(np.int64)
    out = (rank - 1) * int(local_num_gpus) + c_remainder(values, local_num_gpus).astype(np.int64)
    return out.astype(values.dtype)


def split_sizes(sorted_owner, num_owners):
    """The split-size recipe of swap_gradients (python/EmbCache/sparse_optim.py:50-54) and
    test/test_binarysearch2.py:23-27: cudaBinarySearch2(arange(P), sorted owners), then adjacent
    differences."""
    ub = upper_bound(sorted_owner, np.arange(num_owners, dtype=np.asarray(sorted_owner).dtype))
    ub = ub.astype(np.int64)
    ub[1:] = ub[1:] - ub[:-1]
    return ub


def bucket_by_owner(ids, partition_range, local_num_gpus, num_owners, grad=None, cnt=None):
    """The pre-exchange half of swap_gradients (python/EmbCache/sparse_optim.py:33-52): owner of
    every id (cudaReminder without a partition range, cudaBinarySearch with one), sort by owner,
    reorder ids / grads / counts, split sizes.  torch.sort(split) (:41) leaves the order of equal
    owners unspecified; this restatement fixes it as the stable one (input order inside a bucket).
    Returns (ids, grad, cnt, split_sizes, perm)."""
    ids = np.asarray(ids, dtype=np.int64)
    if partition_range is None:
        owner = c_remainder(ids, local_num_gpus)
    else:
        owner = owner_rank(ids, np.asarray(partition_range, dtype=np.int64), local_num_gpus)
    perm = np.argsort(owner, kind="stable").astype(np.int64)
    sizes = split_sizes(owner[perm], num_owners)
    return (ids[perm], None if grad is None else np.asarray(grad)[perm],
            None if cnt is None else np.asarray(cnt)[perm], sizes, perm)


# ---------------------------------------------------------------------------
# lookup against the sorted hot set (closed form over BinarySearchKernel2)
# ---------------------------------------------------------------------------
def lookup_sorted(q, sorted_hot):
    """loc = slot of q in the ascending duplicate-free hot set, or -1.  Built on the reference's
    UpperBound (src/cuda/binary_search.cu:24-33); replaces index_map[q] of
    python/EmbCache/cache.py:163-171 (there: -1 for uncached, arange slot otherwise)."""
    q = np.asarray(q, dtype=np.int64)
    sorted_hot = np.asarray(sorted_hot, dtype=np.int64)
    pos = np.searchsorted(sorted_hot, q, side="right")
    loc = np.full(q.shape, -1, dtype=np.int64)
    if sorted_hot.size:
        prev = sorted_hot[np.maximum(pos - 1, 0)]
        hit = (pos > 0) & (prev == q)
        loc[hit] = pos[hit] - 1
    return loc


def dense_index_map(num_rows, cached_ids, dtype=np.int64):
    """idx_map of python/EmbCache/cache.py:163,170: -1 everywhere, slot number at cached ids."""
    m = np.full(num_rows, -1, dtype=dtype)
    m[np.asarray(cached_ids)] = np.arange(len(cached_ids), dtype=dtype)
    return m


def select_hot_ids(hotness, num_hot, candidate_ids=None):
    """Placement of python/EmbCache/cache.py:165-168: argsort(hotness, descending)[:cached_num].
    Returned ascending.  (Ties are broken however torch.argsort breaks them, as in the reference.)"""
    hotness = torch.as_tensor(hotness)
    if candidate_ids is None:
        candidate_ids = torch.arange(hotness.numel(), dtype=torch.int64)
    order = torch.argsort(hotness[candidate_ids], descending=True)
    return np.sort(candidate_ids[order][:num_hot].numpy().astype(np.int64))


# ---------------------------------------------------------------------------
# split: src/cuda/split.cu
# ---------------------------------------------------------------------------
def split_masks(ids, class_table):
    """_split (src/cuda/split.cu:13-51): three bool masks, mask_k[i] = class_table[ids[i]] == k
    (0 local, 1 remote-hot, 2 remote-cold, :11); other table values set no mask."""
    v = np.asarray(class_table)[np.asarray(ids).astype(np.int64)]
    return v == 0, v == 1, v == 2


def split_compact(loc):
    """hot <=> loc >= 0; compaction as the reference does it with torch.nonzero
    (python/EmbCache/dist_emb.py:179-180): ascending positions of each class."""
    loc = np.asarray(loc)
    hot = loc >= 0
    return hot, np.nonzero(hot)[0].astype(np.int64), np.nonzero(~hot)[0].astype(np.int64)


def split3_compact(ids, class_table):
    masks = split_masks(ids, class_table)
    return masks, tuple(np.nonzero(m)[0].astype(np.int64) for m in masks)


# ---------------------------------------------------------------------------
# row gather / scatter: src/cuda/uva_fetch.cu, src/cuda/uva_set.cu
# ---------------------------------------------------------------------------
def fetch(src, src_index, dst, dst_index):
    """UVAFetchKernel (src/cuda/uva_fetch.cu:11-26): dst[dst_index[i]] = src[src_index[i]], in place."""
    dst[np.asarray(dst_index).astype(np.int64)] = src[np.asarray(src_index).astype(np.int64)]
    return dst


def fetch2(src, src_index):
    """UVAFetchKernel2 / UVAFetch1DKernel2 (src/cuda/uva_fetch.cu:48-70): dst[i] = src[src_index[i]]."""
    return np.asarray(src)[np.asarray(src_index).astype(np.int64)].copy()


def fetch_with_cache2(cpu_src, gpu_src, src_index, index_map):
    """CUDAFetchWithCacheKernel2 (src/cuda/uva_fetch.cu:108-130):
    g = index_map[idx]; dst[i] = gpu_src[g] if g != -1 else cpu_src[idx]."""
    idx = np.asarray(src_index).astype(np.int64)
    g = np.asarray(index_map)[idx].astype(np.int64)
    out = np.asarray(cpu_src)[idx].copy()
    hit = g != -1
    out[hit] = np.asarray(gpu_src)[g[hit]]
    return out


def set_rows(src, dst, dst_index):
    """UVASetKernel / UVACombineKernel (src/cuda/uva_set.cu:11-24, src/cuda/uva_fetch.cu:195-210):
    dst[dst_index[i]] = src[i], in place (indices unique in every caller)."""
    di = np.asarray(dst_index).astype(np.int64)
    dst[di] = np.asarray(src)[: di.size]
    return dst


def set_with_cache(src, cpu_dst, gpu_dst, dst_index, index_map):
    """CUDASetWithCacheKernel (src/cuda/uva_set.cu:71-93): the row goes to gpu_dst[g] when
    g = index_map[idx] != -1, else to cpu_dst[idx].  In place on both."""
    idx = np.asarray(dst_index).astype(np.int64)
    g = np.asarray(index_map)[idx].astype(np.int64)
    hit = g != -1
    src = np.asarray(src)[: idx.size]
    gpu_dst[g[hit]] = src[hit]
    cpu_dst[idx[~hit]] = src[~hit]
    return cpu_dst, gpu_dst


def cached_fetch(cold, hot, q, sorted_hot):
    """cached_fetch keyed by the sorted hot set = fetch_with_cache2 with index_map replaced by the
    binary search (same select: src/cuda/uva_fetch.cu:118-128)."""
    q = np.asarray(q, dtype=np.int64)
    loc = lookup_sorted(q, sorted_hot)
    out = np.asarray(cold)[q].copy()
    hit = loc >= 0
    out[hit] = np.asarray(hot)[loc[hit]]
    return out


def cached_set(src, cold, hot, q, sorted_hot):
    q = np.asarray(q, dtype=np.int64)
    loc = lookup_sorted(q, sorted_hot)
    hit = loc >= 0
    src = np.asarray(src)[: q.size]
    hot[loc[hit]] = src[hit]
    cold[q[~hit]] = src[~hit]
    return cold, hot


# ---------------------------------------------------------------------------
# the split schedule: split first, then one gather / update per class
# (python/EmbCache/dist_emb.py:174-211: cudaSplit, torch.nonzero per class, one cudaFetch per class
# into the positions of that class)
# ---------------------------------------------------------------------------
def lookup_split(q, sorted_hot, num_live=None):
    """(loc, hot_pos, cold_pos): slot of every query, ascending positions of each class; entries
    at and beyond num_live are in neither list and keep loc as computed for the live ones only."""
    q = np.asarray(q, dtype=np.int64)
    live = q.size if num_live is None else max(0, min(int(num_live), q.size))
    loc = lookup_sorted(q[:live], sorted_hot)
    _, hot_pos, cold_pos = split_compact(loc)
    return loc, hot_pos, cold_pos


def fetch_listed(table, index, pos_list, count, out):
    """out[p] = table[index[p]] for the first `count` positions of pos_list (cudaFetch with
    dst_index = the positions of one class, python/EmbCache/dist_emb.py:205-211); in place."""
    pos = np.asarray(pos_list, dtype=np.int64)[: max(0, int(count))]
    out[pos] = np.asarray(table)[np.asarray(index, dtype=np.int64)[pos]]
    return out


def set_listed(src, table, index, pos_list, count):
    """table[index[p]] = src[p] for the first `count` positions of pos_list; in place."""
    pos = np.asarray(pos_list, dtype=np.int64)[: max(0, int(count))]
    table[np.asarray(index, dtype=np.int64)[pos]] = np.asarray(src)[pos]
    return table


def fetch_split(cold, hot, q, sorted_hot):
    """cached_fetch done class by class; must equal cached_fetch."""
    q = np.asarray(q, dtype=np.int64)
    loc, hot_pos, cold_pos = lookup_split(q, sorted_hot)
    out = np.empty((q.size,) + np.asarray(hot).shape[1:], dtype=np.asarray(hot).dtype)
    fetch_listed(hot, loc, hot_pos, hot_pos.size, out)
    fetch_listed(cold, q, cold_pos, cold_pos.size, out)
    return out


def adagrad_listed(row_index, grad, pos_list, count, w, s, lr, eps):
    """adagrad_rows on the rows row_index[p] of (w, s) with gradient grad[p], p over the first
    `count` positions of pos_list; in place."""
    pos = np.asarray(pos_list, dtype=np.int64)[: max(0, int(count))]
    rows = np.asarray(row_index, dtype=np.int64)[pos]
    w1, s1 = adagrad_rows(w[rows], s[rows], np.asarray(grad)[pos], lr, eps)
    w[rows] = w1
    s[rows] = s1


def adam_listed(row_index, grad, pos_list, count, w, step, m, v, lr, beta1, beta2, eps):
    """adam_rows on the rows row_index[p] of (w, step, m, v) with gradient grad[p], p over the
    first `count` positions of pos_list; in place (the per-class form of
    python/EmbCache/sparse_optim.py:590-685)."""
    pos = np.asarray(pos_list, dtype=np.int64)[: max(0, int(count))]
    rows = np.asarray(row_index, dtype=np.int64)[pos]
    if rows.size == 0:
        return
    w[rows], step[rows], m[rows], v[rows] = adam_rows(w[rows], step[rows], m[rows], v[rows],
                                                      np.asarray(grad)[pos], lr, beta1, beta2, eps)


def sparse_adagrad_step_split(cold_w, cold_s, hot_w, hot_s, sorted_hot, uids, g, lr, eps,
                              num_live=None):
    """sparse_adagrad_step done class by class; must equal sparse_adagrad_step."""
    loc, hot_pos, cold_pos = lookup_split(uids, sorted_hot, num_live)
    adagrad_listed(loc, g, hot_pos, hot_pos.size, hot_w, hot_s, lr, eps)
    adagrad_listed(uids, g, cold_pos, cold_pos.size, cold_w, cold_s, lr, eps)


def class_ordered_keys(q, sorted_hot, key_bits):
    """Sort key of every query for the keyed step: the id if cold, (1 << key_bits) | slot if hot.
    Ascending keys = the cold ids in id order, then the hot ids in slot order (= id order)."""
    q = np.asarray(q, dtype=np.int64)
    loc = lookup_sorted(q, sorted_hot)
    return np.where(loc >= 0, (np.int64(1) << np.int64(key_bits)) | loc, q).astype(np.int64)


def averaged(sums, cnts, average):
    """The division of unique_grads (python/EmbCache/sparse_optim.py:142-157): per-id sums over
    their occurrence counts ("mean", :150-156), or over one more ("one_plus": with a count vector
    of ones the reference's divisor is 1 + the occurrences, :145-148), in float32 as torch does
    it (float32 tensor / int64 tensor).  None returns the sums."""
    if average in (None, "sum"):
        return sums
    div = cnts.astype(np.int64) + (1 if average == "one_plus" else 0)
    return (sums / div.astype(np.float32)[:, None]).astype(np.float32)


def keyed_step(cold_w, cold_s, hot_w, hot_s, sorted_hot, q, grad, lr, eps, key_bits,
               fetched_rows=None, average=None):
    """One combine + Adagrad step done the keyed way: combine over the class-ordered keys
    (only_unique_grads arithmetic, python/EmbCache/sparse_optim.py:132-139, on another key), then
    the cold runs update the cold tables at row = key and the hot runs the hot tables at row =
    key minus the class bit.  In place.  Must equal combine_sequential on the ids followed by
    sparse_adagrad_step.  With fetched_rows (one row per query, what the forward pass fetched) the
    old weight of a cold run is the fetched row of its first occurrence instead of the table row.
    Returns (ukeys, sums, cnts, first hot run)."""
    keys = class_ordered_keys(q, sorted_hot, key_bits)
    ukeys, sums, cnts = combine_sequential(keys, grad)
    applied = averaged(sums, cnts, average)
    thr = np.int64(1) << np.int64(key_bits)
    split = int(np.searchsorted(ukeys, thr, side="left"))
    rows = ukeys[:split]
    old = cold_w[rows]
    if fetched_rows is not None:
        first = np.array([np.flatnonzero(keys == k)[0] for k in rows], dtype=np.int64)
        old = np.asarray(fetched_rows)[first] if rows.size else old
    w1, s1 = adagrad_rows(old, cold_s[rows], applied[:split], lr, eps)
    cold_w[rows], cold_s[rows] = w1, s1
    slots = ukeys[split:] - thr
    w1, s1 = adagrad_rows(hot_w[slots], hot_s[slots], applied[split:], lr, eps)
    hot_w[slots], hot_s[slots] = w1, s1
    return ukeys, sums, cnts, split


def keyed_step_adam(cold, hot, sorted_hot, q, grad, lr, beta1, beta2, eps, key_bits,
                    fetched_rows=None, average=None):
    """keyed_step with the reference's SparseAdam arithmetic (adam_rows) in place of Adagrad.
    `cold` and `hot` are (w, step, m, v) table sets, updated in place.  Must equal
    combine_sequential on the ids followed by adam_rows on the gathered rows of each id.
    Returns (ukeys, sums, cnts, first hot run)."""
    keys = class_ordered_keys(q, sorted_hot, key_bits)
    ukeys, sums, cnts = combine_sequential(keys, grad)
    applied = averaged(sums, cnts, average)
    thr = np.int64(1) << np.int64(key_bits)
    split = int(np.searchsorted(ukeys, thr, side="left"))
    for tabs, rows, g, is_cold in ((cold, ukeys[:split], applied[:split], True),
                                   (hot, ukeys[split:] - thr, applied[split:], False)):
        if rows.size == 0:
            continue
        w, step, m, v = tabs
        old = w[rows]
        if is_cold and fetched_rows is not None:
            first = np.array([np.flatnonzero(keys == k)[0] for k in rows], dtype=np.int64)
            old = np.asarray(fetched_rows)[first]
        w[rows], step[rows], m[rows], v[rows] = adam_rows(old, step[rows], m[rows], v[rows], g,
                                                          lr, beta1, beta2, eps)
    return ukeys, sums, cnts, split


# ---------------------------------------------------------------------------
# combine: python/EmbCache/sparse_optim.py:132-157
# ---------------------------------------------------------------------------
def only_unique_grads(idx, grad):
    """The reference's code verbatim in behaviour (python/EmbCache/sparse_optim.py:132-139):
    torch.unique(return_inverse, return_counts) then zeros(float32).index_add_.  torch CPU tensors
    in, torch CPU tensors out."""
    idx = torch.as_tensor(idx)
    grad = torch.as_tensor(grad)
    grad_indices, inverse, grad_cnt = torch.unique(idx, return_inverse=True, return_counts=True)
    grad_values = torch.zeros((grad_indices.shape[0], grad.shape[1]))
    grad_values.index_add_(0, inverse, grad)
    return grad_indices, grad_values, grad_cnt


def unique_grads(idx, grad, cnt=None):
    """python/EmbCache/sparse_optim.py:142-157, including the count that starts from ones when a
    cnt vector is given (:145-148)."""
    idx = torch.as_tensor(idx)
    grad = torch.as_tensor(grad)
    if cnt is not None:
        cnt = torch.as_tensor(cnt)
        grad_indices, inverse = torch.unique(idx, return_inverse=True)
        grad_cnt = torch.ones((grad_indices.shape[0],), dtype=cnt.dtype)
        grad_cnt.index_add_(0, inverse, cnt)
    else:
        grad_indices, inverse, grad_cnt = torch.unique(idx, return_inverse=True, return_counts=True)
    grad_values = torch.zeros((grad_indices.shape[0], grad.shape[1]))
    grad_values.index_add_(0, inverse, grad)
    grad_values = grad_values / grad_cnt.unsqueeze(1)
    return grad_indices, grad_values


def combine_sequential(idx, grad):
    """Independent numpy restatement of only_unique_grads: stable sort by id, then a strictly
    sequential float32 sum ((0 + g1) + g2) + ... of each id's rows in occurrence order - the order
    CPU index_add_ adds them in.  Used to cross-check the torch form and as the bit-exact target of
    the deterministic-order mode."""
    idx = np.asarray(idx, dtype=np.int64)
    grad = np.asarray(grad, dtype=np.float32)
    order = np.argsort(idx, kind="stable")
    sidx = idx[order]
    if sidx.size == 0:
        return (np.zeros(0, np.int64), np.zeros((0, grad.shape[1]), np.float32), np.zeros(0, np.int64))
    starts = np.nonzero(np.concatenate(([True], sidx[1:] != sidx[:-1])))[0]
    ends = np.concatenate((starts[1:], [sidx.size]))
    uids = sidx[starts]
    cnts = (ends - starts).astype(np.int64)
    sums = np.zeros((uids.size, grad.shape[1]), dtype=np.float32)
    # add the k-th occurrence of every id that has one, k = 0, 1, 2, ...: each row of `sums`
    # still receives its rows one at a time in occurrence order
    live = np.arange(uids.size)
    k = 0
    while live.size:
        sums[live] = sums[live] + grad[order[starts[live] + k]]
        k += 1
        live = live[cnts[live] > k]
    return uids, sums, cnts


def combine_float64(idx, grad):
    """Reference sums in float64 (for the tolerance mode)."""
    idx = np.asarray(idx, dtype=np.int64)
    uids, inverse, cnts = np.unique(idx, return_inverse=True, return_counts=True)
    sums = np.zeros((uids.size, np.asarray(grad).shape[1]), dtype=np.float64)
    np.add.at(sums, inverse, np.asarray(grad, dtype=np.float64))
    return uids, sums, cnts.astype(np.int64)


# ---------------------------------------------------------------------------
# row optimizers
# ---------------------------------------------------------------------------
def adagrad_rows(w, s, g, lr, eps):
    """Sparse Adagrad on gathered rows, float32, one rounding per operation, in torch's order
    (torch.optim.Adagrad: state_sum.addcmul_(g, g); std = state_sum.sqrt().add_(eps);
    param.addcdiv_(g, std, value=-lr)).  The reference has no Adagrad (its optimizer is SparseAdam,
    python/EmbCache/sparse_optim.py:531); this is the optimizer the benchmark configurations name.
    Returns (w_new, s_new)."""
    w = np.asarray(w, dtype=np.float32)
    s = np.asarray(s, dtype=np.float32)
    g = np.asarray(g, dtype=np.float32)
    lr = np.float32(lr)
    eps = np.float32(eps)
    s1 = (s + g * g).astype(np.float32)
    std = (np.sqrt(s1) + eps).astype(np.float32)
    w1 = (w - (lr * g) / std).astype(np.float32)
    return w1, s1


def sparse_adagrad_step(cold_w, cold_s, hot_w, hot_s, sorted_hot, uids, g, lr, eps):
    """Gather (cached_fetch), adagrad_rows, scatter back (cached_set); in place."""
    w = cached_fetch(cold_w, hot_w, uids, sorted_hot)
    s = cached_fetch(cold_s, hot_s, uids, sorted_hot)
    w1, s1 = adagrad_rows(w, s, g, lr, eps)
    cached_set(w1, cold_w, hot_w, uids, sorted_hot)
    cached_set(s1, cold_s, hot_s, uids, sorted_hot)


def adam_rows(w, step, m, v, g, lr, beta1, beta2, eps):
    """SparseAdam.update arithmetic (python/EmbCache/sparse_optim.py:632-657,681) on gathered rows,
    with torch CPU float32 ops in the reference's order.  Returns (w, step, m, v) new."""
    w, step, m, v, g = (torch.as_tensor(np.asarray(x, dtype=np.float32)) for x in (w, step, m, v, g))
    state_step = step + 1                                                  # :634
    grad_power = g * g                                                     # :640
    update_mem = beta1 * m + (1.0 - beta1) * g                             # :641
    update_power = beta2 * v + (1.0 - beta2) * grad_power                  # :642
    update_mem_corr = update_mem / (1.0 - torch.pow(torch.tensor(beta1), state_step)).unsqueeze(1)    # :652
    update_power_corr = update_power / (1.0 - torch.pow(torch.tensor(beta2), state_step)).unsqueeze(1)  # :654
    std_values = lr * update_mem_corr / (torch.sqrt(update_power_corr) + eps)                           # :656
    w_new = w - std_values                                                 # :681
    return w_new.numpy(), state_step.numpy(), update_mem.numpy(), update_power.numpy()


# ---------------------------------------------------------------------------
# cold-gradient accumulator: python/EmbCache/server.py:546-562 (accumulate), :346-419 (flush)
# ---------------------------------------------------------------------------
class ColdGradAccumulatorModel:
    """Dict model: per unique incoming id  buf[id] += g; cnt[id] += c  (server.py:556-559); flush
    emits every entry with cnt > 0 in ascending id order and resets it (:413-419; the gradient row
    is zeroed too - the reference's `buf[idx][:] = 0` at :414 writes to a temporary copy and is a
    no-op there, the evident intent is what is modelled)."""

    def __init__(self, dim):
        self.dim = dim
        self.rows = {}
        self.cnt = {}

    def accumulate(self, ids, grad, cnt=None):
        ids = np.asarray(ids, dtype=np.int64)
        grad = np.asarray(grad, dtype=np.float32)
        for i, k in enumerate(ids.tolist()):
            c = 1 if cnt is None else int(cnt[i])
            if k in self.rows:
                self.rows[k] = (self.rows[k] + grad[i]).astype(np.float32)
                self.cnt[k] += c
            else:
                self.rows[k] = (np.zeros(self.dim, np.float32) + grad[i]).astype(np.float32)
                self.cnt[k] = c

    def flush(self):
        keys = sorted(self.rows)
        ids = np.array(keys, dtype=np.int64)
        sums = np.stack([self.rows[k] for k in keys]) if keys else np.zeros((0, self.dim), np.float32)
        cnts = np.array([self.cnt[k] for k in keys], dtype=np.int64)
        self.rows, self.cnt = {}, {}
        return ids, sums, cnts


# ---------------------------------------------------------------------------
# set-associative index cache: src/cache/cache.h, src/cache/cache_line.h, src/cache/lookup.cu
# ---------------------------------------------------------------------------
class SACacheIndexModel:
    """SACacheIndex<int64, int64> (src/cache/cache.h:11-259) over 8-entry lines
    (CACHE_LINE_SIZE, src/cache/cache_line.h:5), batches processed in input order (the reference's
    OpenMP loops give that order with one thread; with more, the outcome for ids that share a line
    depends on thread timing).  Pure-Python loops: for small cases.  Ids must be >= 0
    (`id % index_size` indexes the line array, cache.h:27).

    State: ids[line, entry] (-1 = empty) and age[line, entry] (the access table)."""
    LINE = 8

    def __init__(self, cache_size):
        self.lines = (int(cache_size) + self.LINE - 1) // self.LINE       # cache.h:139
        self.ids = np.full((self.lines, self.LINE), -1, dtype=np.int64)    # cache_line.h:13-18
        self.age = np.zeros((self.lines, self.LINE), dtype=np.int32)

    def get_capacity(self):                                               # cache.h:187-189
        return self.lines * self.LINE

    def get_valid_entries_num(self):                                      # cache.h:180-185
        return int((self.ids != -1).sum())

    def _set_id(self, ln, e, v):                                          # cache_line.h:20-24
        self.ids[ln, e] = v
        self.age[ln, e] = 0

    def _find(self, ln, v):                                               # cache_line.h:48-56
        for e in range(self.LINE):
            if self.ids[ln, e] == v:
                return e
        return -1

    def add(self, ids):
        """_add (cache.h:51-91): the id's entry if present; else the LAST empty entry of its line
        (find_or_empty_entry keeps overwriting idx, cache_line.h:66-77); else the entry with the
        largest non-zero age (find_lru, cache_line.h:91-102: strictly greater than entry 0's, so
        ties go to the lowest entry), or -1 when every age is 0."""
        ids = np.asarray(ids, dtype=np.int64)
        locs = np.full(ids.shape, -1, dtype=np.int64)
        for i, v in enumerate(ids.tolist()):
            ln = v % self.lines
            idx, exist = -1, False
            for e in range(self.LINE):
                cur = self.ids[ln, e]
                if cur == v:
                    idx, exist = e, True
                    break
                if cur == -1:
                    idx = e
            if idx >= 0:
                if not exist:
                    self._set_id(ln, idx, v)
                locs[i] = ln * self.LINE + idx                            # compute_loc :31-33
                continue
            lru, tmp = 0, int(self.age[ln, 0])
            for e in range(self.LINE):
                a = int(self.age[ln, e])
                if a > tmp and a != 0:
                    lru, tmp = e, a
            if tmp != 0:
                self._set_id(ln, lru, v)
                locs[i] = ln * self.LINE + lru
        return locs

    def lookup(self, ids):
        """_lookup (cache.h:93-107): loc or -1; a hit ages every entry of the line by one and
        zeroes the hit entry (access_loc, cache_line.h:79-85)."""
        ids = np.asarray(ids, dtype=np.int64)
        locs = np.full(ids.shape, -1, dtype=np.int64)
        for i, v in enumerate(ids.tolist()):
            ln = v % self.lines
            e = self._find(ln, v)
            if e >= 0:
                locs[i] = ln * self.LINE + e
                self.age[ln] += 1
                self.age[ln, e] = 0
        return locs

    def cudalookup(self, ids):
        """lookupkernel2 (src/cache/lookup.cu:15-45): the same search on a copy of the line, so no
        aging; misses keep the -1 the output was filled with (cache.h:222-231)."""
        ids = np.asarray(ids, dtype=np.int64)
        ln = ids % self.lines
        hit = self.ids[ln] == ids[:, None]
        e = hit.argmax(axis=1)
        return np.where(hit.any(axis=1), ln * self.LINE + e, -1).astype(np.int64)

    def reset(self, ids):
        """_reset (cache.h:109-121): an id that is present gives its entry back."""
        for v in np.asarray(ids, dtype=np.int64).tolist():
            ln = v % self.lines
            e = self._find(ln, v)
            if e >= 0:
                self._set_id(ln, e, -1)

    def getall(self, length):
        """_getall (cache.h:123-137): live (id, loc) pairs in line order, at most `length`."""
        flat = self.ids.reshape(-1)
        locs = np.nonzero(flat != -1)[0][:length].astype(np.int64)
        return flat[locs].copy(), locs


class ColdCacheServerModel:
    """Gradient path of EmbCacheServer (python/EmbCache/server.py) with the same torch CPU calls,
    over SACacheIndexModel: _create_cache buffers (:76-166), _update_cache for one client
    (:510-541), _accumulate_gradients_cold_remote (:546-562), _accumulate_gradients_cold_local
    (:564-574) and both halves of _send_staled_gradients (:346-419, :421-497) up to the point
    where rows are handed to the clients.  One deliberate difference: the reference's
    `buf[index][:] = 0` (:414, :489, :537) assigns into a temporary and zeroes nothing; the rows
    are zeroed here (the evident intent)."""

    def __init__(self, cache_size, dim, hotness, cnt_threshold=16, part_start=0, part_nnodes=0):
        hotness = torch.as_tensor(hotness, dtype=torch.float32)
        self.cnt_threshold = int(cnt_threshold)
        self.threshold = (1 / (0.001 + hotness)).ceil().int().clamp(max=100)      # :87-88
        self.index = SACacheIndexModel(cache_size)
        S = self.index.get_capacity()                                              # :98
        self.emb = torch.zeros((S, dim))
        self.grad = torch.zeros((S, dim))                                          # :108-112
        self.cnt = torch.zeros(S, dtype=torch.int32)                               # :115-121
        self.iter = torch.zeros(S, dtype=torch.int32)                              # :124-125
        self.iter_thr = torch.zeros(S, dtype=torch.int32)                          # :127
        self.idx = torch.full((S,), -1, dtype=torch.int64)                         # :132-139
        self.part_start = int(part_start)
        self.l_grad = torch.zeros((part_nnodes, dim))                              # :144-149
        self.l_cnt = torch.zeros(part_nnodes, dtype=torch.int32)                   # :151-157
        self.l_iter = torch.zeros(part_nnodes, dtype=torch.int32)                  # :160-161
        self.l_thr = self.threshold[part_start:part_start + part_nnodes]           # :164-166

    def update_cache(self, ids, embs):
        ids, embs = torch.as_tensor(ids), torch.as_tensor(embs)
        locs = torch.from_numpy(self.index.add(ids.numpy()))                       # :513
        valid_index = torch.nonzero(locs >= 0).flatten()                           # :519-520
        valid_locs = locs[valid_index]
        # an id already cached at a loc and a later id of the batch that evicts it both report
        # that loc; index assignment with a repeated index keeps the row written last, made
        # explicit here (torch leaves the order of repeated indices unspecified)
        _, first_rev = np.unique(valid_locs.numpy()[::-1], return_index=True)
        keep = torch.from_numpy(np.sort(valid_locs.numel() - 1 - first_rev))
        valid_index, valid_locs = valid_index[keep], valid_locs[keep]
        self.emb[valid_locs] = embs[valid_index]                                   # :531
        self.grad[valid_locs] = 0                                                  # :537 (intent)
        self.cnt[valid_locs] = 0                                                   # :538
        self.idx[valid_locs] = -1                                                  # :539
        return locs.numpy()

    def accumulate_gradients_cold_remote(self, id, grad):
        id, grad = torch.as_tensor(id), torch.as_tensor(grad)
        locs = torch.from_numpy(self.index.lookup(id.numpy()))                     # :550
        cache_idx = torch.nonzero(locs >= 0).flatten()                             # :551-552
        if cache_idx.numel() > 0:
            tmp = locs[cache_idx]
            self.idx[tmp] = id[cache_idx]                                          # :556
            self.iter_thr[tmp] = self.threshold[id[cache_idx]]                     # :557
            self.grad[tmp] += grad[cache_idx]                                      # :558
            self.cnt[tmp] += 1                                                     # :559
        return locs.numpy()

    def accumulate_gradients_cold_local(self, id, grad):
        id, grad = torch.as_tensor(id), torch.as_tensor(grad)
        if id.numel() > 0:
            local_id = id - self.part_start                                        # :569
            self.l_grad[local_id] += grad                                          # :570
            self.l_cnt[local_id] += 1                                              # :571

    def _staled(self, grad, cnt, it, thr):
        cnt_index = torch.nonzero(cnt > 0).flatten()                               # :350-351
        mask = (it[cnt_index] >= thr[cnt_index]) | (cnt[cnt_index] >= self.cnt_threshold)  # :352-355
        staled_index = cnt_index[mask]                                             # :357
        out_grads = grad[staled_index].clone()                                     # :362
        out_cnt = cnt[staled_index].long()                                         # :363, sent as int64 (:384-386)
        grad[staled_index] = 0                                                     # :414 (intent)
        cnt[staled_index] = 0                                                      # :415
        it[cnt_index] += 1                                                         # :418
        it[staled_index] = 0                                                       # :419
        return staled_index, out_grads, out_cnt

    def staled_gradients_remote(self):
        staled_index, grads, cnts = self._staled(self.grad, self.cnt, self.iter, self.iter_thr)
        ids = self.idx[staled_index].clone()                                       # :361
        self.index.reset(ids.numpy())                                              # :413
        return ids.numpy(), grads.numpy(), cnts.numpy()

    def staled_gradients_local(self):
        staled_index, grads, cnts = self._staled(self.l_grad, self.l_cnt, self.l_iter, self.l_thr)
        return (staled_index + self.part_start).numpy(), grads.numpy(), cnts.numpy()   # :437


# ---------------------------------------------------------------------------
# the whole step, for smoke tests and the CPU baseline (torch CPU, as the reference's CPU path)
# ---------------------------------------------------------------------------
def torch_step(cold_w, cold_s, hot_w, hot_s, sorted_hot, q, grad, lr, eps):
    """lookup -> cached_fetch -> combine -> sparse Adagrad with torch CPU ops on torch CPU tensors,
    in place on the four tables.  Returns (fetched rows, uids, sums, cnts).  This is the shape the
    reference's CPU-side code has: searchsorted for the lookup, indexed reads, torch.unique +
    index_add_ for the combine (python/EmbCache/sparse_optim.py:132-139), element-wise update."""
    def lookup(ids):
        if sorted_hot.numel() == 0:
            return torch.full_like(ids, -1)
        pos = torch.searchsorted(sorted_hot, ids, right=True)
        prev = sorted_hot[(pos - 1).clamp_(min=0)]
        return torch.where((pos > 0) & (prev == ids), pos - 1, torch.full_like(pos, -1))

    loc = lookup(q)
    hit = loc >= 0
    rows = torch.empty((q.numel(), cold_w.shape[1]), dtype=cold_w.dtype)
    rows[hit] = hot_w[loc[hit]]
    rows[~hit] = cold_w[q[~hit]]

    uids, sums, cnts = only_unique_grads(q, grad)

    uloc = lookup(uids)
    uh = uloc >= 0
    for (w_tab, s_tab, sel, index) in ((hot_w, hot_s, uh, uloc[uh]), (cold_w, cold_s, ~uh, uids[~uh])):
        g = sums[sel]
        s = s_tab[index].addcmul_(g, g, value=1.0)
        std = s.sqrt().add_(eps)
        w = w_tab[index].addcdiv_(g, std, value=-lr)
        s_tab[index] = s
        w_tab[index] = w
    return rows, uids, sums, cnts
