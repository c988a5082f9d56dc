"""Pins the CPU oracle (oracle/hades_oracle.py, oracle/hades_oracle.c) against library routines,
brute force, closed forms and the recipes held by the reference's own test scripts.  No GPU."""
import bisect
import ctypes

import numpy as np
import pytest
import torch

from oracle import hades_oracle as O

RNG = np.random.default_rng(20251125)


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


# ---- routing ---------------------------------------------------------------------
def test_upper_bound_matches_bisect_and_edges():
    rng = np.random.default_rng(1)
    r = np.sort(rng.integers(-50, 50, size=40)).astype(np.int64)  # duplicates allowed in a range
    v = rng.integers(-60, 60, size=300).astype(np.int64)
    want = np.array([bisect.bisect_right(r.tolist(), x) for x in v.tolist()], dtype=np.int64)
    assert np.array_equal(O.upper_bound(r, v), want)
    assert O.upper_bound(np.zeros(0, np.int64), v).sum() == 0          # empty range
    assert O.upper_bound(r, np.array([r[0] - 1]))[0] == 0              # below the minimum
    assert O.upper_bound(r, np.array([r[-1]]))[0] == r.size            # equal to the maximum
    assert O.upper_bound(r.astype(np.int32), v.astype(np.int32)).dtype == np.int32


def test_reminder_is_c_remainder():
    v = np.array([7, -7, 0, 12345678901, -1], dtype=np.int64)
    want = np.array([int(np.fmod(x, 4)) for x in v], dtype=np.int64)
    assert np.array_equal(O.c_remainder(v, 4), want)
    assert list(O.c_remainder(v, 4)) == [3, -3, 0, 12345678901 % 4, -1]


def test_owner_rank_and_split_sizes_recipe():
    # the recipe printed by test/test_binarysearch2.py:6-27, with an assertion added:
    # ids in [0, 3M), 2 partitions x 4 local GPUs, then split sizes by sorted owner
    num_part, local = 2, 4
    rng = np.random.default_rng(2)
    index = rng.integers(0, 3_000_000, size=1000).astype(np.int64)
    range_partition = np.array([i * 3_000_000 // num_part for i in range(num_part + 1)], np.int64)
    owner = O.owner_rank(index, range_partition, local)
    want = np.array([(bisect.bisect_right(range_partition.tolist(), x) - 1) * local + x % local
                     for x in index.tolist()], dtype=np.int64)
    assert np.array_equal(owner, want)
    assert owner.min() >= 0 and owner.max() < num_part * local
    sizes = O.split_sizes(np.sort(owner), num_part * local)
    assert np.array_equal(sizes, np.bincount(owner, minlength=num_part * local))
    assert sizes.sum() == index.size


@pytest.mark.parametrize("ranged", [False, True])
def test_bucket_by_owner_is_the_reference_recipe_made_stable(ranged):
    # swap_gradients (python/EmbCache/sparse_optim.py:33-52) with torch's own sort, stable
    rng = np.random.default_rng(21)
    num_part, local = (3, 4) if ranged else (1, 8)
    ids = rng.integers(0, 90_000, size=5000).astype(np.int64)
    grad = rng.standard_normal((ids.size, 4)).astype(np.float32)
    cnt = rng.integers(1, 9, ids.size).astype(np.int64)
    rp = np.array([i * 90_000 // num_part for i in range(num_part + 1)], np.int64) if ranged else None
    G = num_part * local
    b_ids, b_grad, b_cnt, sizes, perm = O.bucket_by_owner(ids, rp, local, G, grad, cnt)
    split = torch.from_numpy(O.owner_rank(ids, rp, local) if ranged else O.c_remainder(ids, local))
    value, indices = torch.sort(split, stable=True)
    assert np.array_equal(perm, indices.numpy())
    assert np.array_equal(b_ids, ids[indices.numpy()]) and np.array_equal(b_grad, grad[indices.numpy()])
    assert np.array_equal(b_cnt, cnt[indices.numpy()])
    assert np.array_equal(sizes, torch.bincount(split, minlength=G).numpy())
    # brute force: bucket g holds exactly the rows owned by g, in input order
    start = 0
    for g in range(G):
        rows = [i for i in range(ids.size) if int(split[i]) == g]
        assert perm[start:start + len(rows)].tolist() == rows
        start += len(rows)
    assert start == ids.size


# ---- lookup -----------------------------------------------------------------------
def test_lookup_sorted_brute_force_and_edges():
    rng = np.random.default_rng(3)
    hot = np.sort(rng.choice(500, size=60, replace=False)).astype(np.int64)
    q = rng.integers(-5, 510, size=400).astype(np.int64)
    eq = q[:, None] == hot[None, :]
    want = np.where(eq.any(1), eq.argmax(1), -1)
    assert np.array_equal(O.lookup_sorted(q, hot), want)
    assert np.array_equal(O.lookup_sorted(q, np.zeros(0, np.int64)), np.full(q.size, -1))
    assert np.array_equal(O.lookup_sorted(np.array([hot[0], hot[-1], hot[0] - 1, hot[-1] + 1]), hot),
                          [0, hot.size - 1, -1, -1])
    # agrees with the dense index_map of the reference (cache.py:163,170)
    m = O.dense_index_map(600, hot)
    qq = q[(q >= 0) & (q < 600)]
    assert np.array_equal(O.lookup_sorted(qq, hot), m[qq])


def test_select_hot_ids_is_topk_by_hotness():
    hotness = torch.tensor([0.1, 5.0, 3.0, 9.0, 0.0, 4.0])
    assert list(O.select_hot_ids(hotness, 3)) == [1, 3, 5]
    assert list(O.select_hot_ids(hotness, 0)) == []
    cand = torch.tensor([0, 2, 4, 5])
    assert list(O.select_hot_ids(hotness, 2, cand)) == [2, 5]


# ---- split ------------------------------------------------------------------------
def test_split_matches_reference_cpu_recipe():
    # test/test_split.py:9-37: hot/remote masks -> int8 class table -> boolean-mask split on CPU
    torch.manual_seed(42)
    n_nodes = 20_000
    remote = torch.zeros(n_nodes).bool()
    remote[torch.randint(0, n_nodes, (n_nodes // 2,))] = True
    hot = torch.zeros(n_nodes).bool()
    hot[torch.randint(0, n_nodes, (n_nodes // 2,))] = True
    total = torch.zeros(n_nodes).char()
    total[hot & remote] = 1
    total[(~hot) & remote] = 2
    index = torch.randint(0, n_nodes, (5000,))
    local_m, rhot_m, rcold_m = O.split_masks(index.numpy(), total.numpy())
    assert np.array_equal(rhot_m, (hot & remote)[index].numpy())
    assert np.array_equal(rcold_m, ((~hot) & remote)[index].numpy())
    assert np.array_equal(local_m, (~remote)[index].numpy())
    assert np.array_equal(local_m ^ rhot_m ^ rcold_m, np.ones(5000, bool))   # disjoint cover
    assert not (local_m & rhot_m).any() and not (rhot_m & rcold_m).any()
    # a class value outside {0,1,2} sets no mask (split.cu:37-43 has no else branch)
    t2 = total.numpy().copy()
    t2[index[0]] = 5
    a, b, c = O.split_masks(index.numpy(), t2)
    assert not (a[0] or b[0] or c[0])


def test_split_compact_is_nonzero():
    loc = np.array([3, -1, -1, 0, 7, -1], dtype=np.int64)
    hot, hp, cp = O.split_compact(loc)
    assert list(hot) == [True, False, False, True, True, False]
    assert list(hp) == [0, 3, 4] and list(cp) == [1, 2, 5]
    assert hp.size + cp.size == loc.size


# ---- gather / scatter: the reference's test recipes ------------------------------------
def _cache_case(rng, n_rows=4000, n_cached=2000, n_q=500, dim=8, dtype=np.float32):
    # test/test_cached_fetch.py:8-17 scaled down
    src = rng.standard_normal((n_rows, dim)).astype(dtype)
    cached_idx = rng.permutation(n_cached).astype(np.int64)
    idx_map = np.full(n_rows, -1, np.int64)
    idx_map[cached_idx] = np.arange(n_cached)
    gpu_src = src[cached_idx].copy()
    q = rng.permutation(n_rows)[:n_q].astype(np.int64)
    return src, gpu_src, idx_map, q


def test_fetch_recipes_bit_exact():
    rng = np.random.default_rng(4)
    src, gpu_src, idx_map, q = _cache_case(rng)
    a = src[q]                                                    # test_cached_fetch.py:22
    assert np.array_equal(O.fetch_with_cache2(src, gpu_src, q, idx_map), a)   # :43, :60
    assert np.array_equal(O.fetch2(src, q), a)                    # :74
    # cached rows really come from the cache copy: poison the host copy of cached rows
    poisoned = src.copy()
    poisoned[idx_map != -1] = np.nan
    assert np.array_equal(O.fetch_with_cache2(poisoned, gpu_src, q, idx_map), a)
    # test/test_fetch.py:16: dst[dst_index] = src[src_index]
    dst = rng.standard_normal((400, 8)).astype(np.float32)
    want = dst.copy()
    di = rng.permutation(400)[:100]
    si = rng.permutation(4000)[:100]
    want[di] = src[si]
    assert np.array_equal(O.fetch(src, si, dst, di), want)
    # 1-D (test_cached_fetch_1D.py)
    s1 = src[:, 0].copy()
    assert np.array_equal(O.fetch_with_cache2(s1, gpu_src[:, 0].copy(), q, idx_map), s1[q])


def test_set_recipes_bit_exact():
    rng = np.random.default_rng(5)
    dst, gpu_dst, idx_map, q = _cache_case(rng)
    src = rng.standard_normal((q.size, 8)).astype(np.float32)
    want = dst.copy()
    want[q] = src                                                  # test_cached_set.py:22
    d1 = dst.copy()
    O.set_rows(src, d1, q)                                         # cudaSet / cudaCombine
    assert np.array_equal(d1[q], want[q]) and np.array_equal(d1, want)
    d2, g2 = dst.copy(), gpu_dst.copy()
    O.set_with_cache(src, d2, g2, q, idx_map)                      # :54-58
    # read back through the cache: equals the plain scatter on the touched rows
    assert np.array_equal(O.fetch_with_cache2(d2, g2, q, idx_map), want[q])
    # and only the live copy was written
    hit = idx_map[q] != -1
    assert np.array_equal(d2[q[hit]], dst[q[hit]])


def test_cached_fetch_sorted_equals_map_form():
    rng = np.random.default_rng(6)
    n_rows, dim = 3000, 4
    cold = rng.standard_normal((n_rows, dim)).astype(np.float32)
    hot_ids = np.sort(rng.choice(n_rows, 700, replace=False)).astype(np.int64)
    hot = cold[hot_ids] + 1.0       # distinguishable
    q = rng.integers(0, n_rows, 900).astype(np.int64)
    m = O.dense_index_map(n_rows, hot_ids)
    assert np.array_equal(O.cached_fetch(cold, hot, q, hot_ids), O.fetch_with_cache2(cold, hot, q, m))


# ---- combine ---------------------------------------------------------------------------
def _zipfish(rng, n, n_ids):
    return np.minimum((rng.pareto(0.9, n)).astype(np.int64), n_ids - 1)


def test_combine_torch_equals_sequential_numpy_bit_exact():
    # index_add_ on CPU adds rows in occurrence order: a stable sort plus a left-to-right float32
    # sum reproduces it bit for bit (also with several intra-op threads)
    rng = np.random.default_rng(7)
    idx = _zipfish(rng, 20000, 300)
    grad = (rng.standard_normal((20000, 16)) * 1e-3).astype(np.float32)
    for threads in (1, 4):
        torch.set_num_threads(threads)
        tu, ts, tc = O.only_unique_grads(torch.from_numpy(idx), torch.from_numpy(grad))
        nu, ns, nc = O.combine_sequential(idx, grad)
        assert np.array_equal(tu.numpy(), nu) and np.array_equal(tc.numpy(), nc)
        assert np.array_equal(ts.numpy(), ns)
    assert ts.dtype == torch.float32
    # against float64 sums
    du, ds, dc = O.combine_float64(idx, grad)
    assert np.array_equal(du, nu) and np.array_equal(dc, nc)
    assert np.abs(ns - ds).max() <= 1e-5 * np.abs(ds).max()


def test_combine_closed_forms_and_invariants():
    rng = np.random.default_rng(8)
    n, d = 257, 8
    grad = rng.standard_normal((n, d)).astype(np.float32)
    # all distinct: output = input permuted by argsort, counts all one
    idx = rng.permutation(10 * n)[:n].astype(np.int64)
    u, s, c = O.combine_sequential(idx, grad)
    order = np.argsort(idx)
    assert np.array_equal(u, idx[order]) and np.array_equal(s, grad[order]) and (c == 1).all()
    # all equal: one row = sequential column sum, count n
    u, s, c = O.combine_sequential(np.full(n, 42, np.int64), grad)
    acc = np.zeros(d, np.float32)
    for r in grad:
        acc = acc + r
    assert list(u) == [42] and list(c) == [n] and np.array_equal(s[0], acc)
    # invariants on a skewed batch
    idx = _zipfish(rng, 5000, 100)
    g = rng.standard_normal((5000, d)).astype(np.float32)
    u, s, c = O.combine_sequential(idx, g)
    assert c.sum() == 5000 and (np.diff(u) > 0).all()
    assert np.allclose(s.sum(0), g.sum(0), rtol=1e-4, atol=1e-3)
    # empty
    u, s, c = O.combine_sequential(np.zeros(0, np.int64), np.zeros((0, d), np.float32))
    assert u.size == 0 and s.shape == (0, d) and c.size == 0
    # -0.0 handling: 0.0f + (-0.0f) = +0.0f
    u, s, c = O.combine_sequential(np.array([1]), np.array([[-0.0]], np.float32))
    assert not np.signbit(s[0, 0])


def test_local_aggregation_is_combine_of_concatenation():
    # combine(concat(batches)) == combine(concat(combine(batch_t))) on ids; counts add up
    rng = np.random.default_rng(9)
    batches = [(_zipfish(rng, 3000, 500), rng.standard_normal((3000, 4)).astype(np.float32))
               for _ in range(4)]
    idx = np.concatenate([b[0] for b in batches])
    g = np.concatenate([b[1] for b in batches])
    u, s, c = O.combine_sequential(idx, g)
    parts = [O.combine_sequential(*b) for b in batches]
    u2, s2, _ = O.combine_sequential(np.concatenate([p[0] for p in parts]),
                                     np.concatenate([p[1] for p in parts]))
    assert np.array_equal(u, u2)
    assert np.allclose(s, s2, rtol=1e-5, atol=1e-6)
    cc = np.zeros(u.size, np.int64)
    for p in parts:
        cc[np.searchsorted(u, p[0])] += p[2]
    assert np.array_equal(cc, c)


def test_unique_grads_mean_and_count_quirk():
    idx = torch.tensor([5, 3, 5, 5, 3])
    grad = torch.tensor([[1.0], [2.0], [3.0], [5.0], [4.0]])
    u, m = O.unique_grads(idx, grad)
    assert u.tolist() == [3, 5] and m.flatten().tolist() == [3.0, 3.0]
    # with cnt: divisor = 1 + sum(cnt) (sparse_optim.py:145-148)
    u, m = O.unique_grads(idx, grad, cnt=torch.tensor([1, 1, 1, 1, 1]))
    assert m.flatten().tolist() == [6.0 / 3, 9.0 / 4]


def test_averaged_is_the_division_of_unique_grads():
    """O.averaged restates the last line of unique_grads (python/EmbCache/sparse_optim.py:156)
    on top of the sequential sums: pinned bit for bit by the reference's own torch code
    (O.unique_grads: unique + index_add_ + division), for the plain mean and for the count that
    starts from ones when a count vector of ones comes along (:145-148); and a keyed step with
    `average` equals combine -> that division -> Adagrad on the ids."""
    rng = np.random.default_rng(91)
    n, D, N = 6000, 5, 900
    q = np.minimum(rng.pareto(0.7, n).astype(np.int64) * 13 % N, N - 1)
    g = (rng.standard_normal((n, D)) * 1e-2).astype(np.float32)
    wu, ws, wc = O.combine_sequential(q, g)
    assert wc.max() > 100                                    # divisors beyond small integers
    tu, tm = O.unique_grads(torch.from_numpy(q), torch.from_numpy(g))
    assert np.array_equal(tu.numpy(), wu) and np.array_equal(tm.numpy(), O.averaged(ws, wc, "mean"))
    tu, tm = O.unique_grads(torch.from_numpy(q), torch.from_numpy(g), cnt=torch.ones(n, dtype=torch.int64))
    assert np.array_equal(tm.numpy(), O.averaged(ws, wc, "one_plus"))
    assert O.averaged(ws, wc, None) is ws
    # closed forms: n copies of one row average to that row; a single occurrence is unchanged
    row = g[:1]
    same = O.averaged(*O.combine_sequential(np.zeros(64, np.int64), np.repeat(row, 64, 0))[1:], "mean")
    assert np.allclose(same, row, rtol=1e-6) and np.array_equal(O.averaged(ws[wc == 1], wc[wc == 1], "mean"), ws[wc == 1])
    # keyed step with the mean = combine, divide, update on the ids
    H, kb = 120, 10
    cold = rng.standard_normal((N, D)).astype(np.float32)
    hot_ids = np.sort(rng.choice(N, H, replace=False)).astype(np.int64)
    for avg in ("mean", "one_plus"):
        a = [cold.copy(), np.zeros((N, D), np.float32), cold[hot_ids] + 1, np.zeros((H, D), np.float32)]
        b = [x.copy() for x in a]
        for _ in range(2):
            O.sparse_adagrad_step(a[0], a[1], a[2], a[3], hot_ids, wu, O.averaged(ws, wc, avg), 0.01, 1e-10)
            O.keyed_step(b[0], b[1], b[2], b[3], hot_ids, q, g, 0.01, 1e-10, kb, average=avg)
        for x, y in zip(a, b):
            assert np.array_equal(x, y)


# ---- optimizers --------------------------------------------------------------------------
def test_adagrad_matches_torch_optim():
    rng = np.random.default_rng(10)
    w0 = (rng.standard_normal((300, 16)) * 0.01).astype(np.float32)
    p = torch.nn.Parameter(torch.from_numpy(w0.copy()))
    opt = torch.optim.Adagrad([p], lr=0.01, eps=1e-10)
    w, s = w0.copy(), np.zeros_like(w0)
    for step in range(3):
        g = (rng.standard_normal(w0.shape) * 1e-3).astype(np.float32)
        p.grad = torch.from_numpy(g.copy())
        opt.step()
        w, s = O.adagrad_rows(w, s, g, 0.01, 1e-10)
        # tolerance of the update parity: 1e-5 relative (bit-exact unless the torch build fuses)
        assert np.allclose(w, p.detach().numpy(), rtol=1e-5, atol=1e-8)
        assert np.allclose(s, opt.state[p]["sum"].numpy(), rtol=1e-6, atol=0)


def test_adagrad_special_cases():
    w = np.array([[0.5, -0.25]], np.float32)
    s = np.array([[0.0, 4.0]], np.float32)
    w1, s1 = O.adagrad_rows(w, s, np.zeros_like(w), 0.01, 1e-10)        # g = 0: w unchanged
    assert np.array_equal(w1, w) and np.array_equal(s1, s)
    g = np.array([[2.0, -3.0]], np.float32)                               # s = 0: step = lr*sign(g)
    w1, s1 = O.adagrad_rows(np.zeros_like(g), np.zeros_like(g), g, 0.01, 1e-10)
    assert np.allclose(w1, -0.01 * np.sign(g), rtol=1e-6) and np.array_equal(s1, g * g)
    # a wrong sign or a dropped sqrt would fail this one: s=9 -> std=3 (+eps), w -= lr*g/3
    w1, _ = O.adagrad_rows(np.ones((1, 1), np.float32), np.full((1, 1), 5.0, np.float32),
                           np.full((1, 1), 2.0, np.float32), 0.3, 0.0)
    assert np.allclose(w1, 1.0 - 0.3 * 2.0 / 3.0, rtol=1e-6)


def test_adam_matches_torch_optim_adam():
    rng = np.random.default_rng(11)
    w0 = (rng.standard_normal((50, 8)) * 0.01).astype(np.float32)
    p = torch.nn.Parameter(torch.from_numpy(w0.copy()))
    opt = torch.optim.Adam([p], lr=0.01, betas=(0.9, 0.999), eps=1e-8)
    w = w0.copy()
    step = np.zeros(50, np.float32)
    m = np.zeros_like(w0)
    v = np.zeros_like(w0)
    for _ in range(4):
        g = (rng.standard_normal(w0.shape) * 1e-2).astype(np.float32)
        p.grad = torch.from_numpy(g.copy())
        opt.step()
        w, step, m, v = O.adam_rows(w, step, m, v, g, 0.01, 0.9, 0.999, 1e-8)
        # the reference forms 1 - beta^step in float32 (sparse_optim.py:652-655): 1 - 0.999 carries a
        # relative error near 6e-5 that torch.optim.Adam (Python doubles) does not have, so the two
        # agree to about 1e-4 of one update (lr), not to 1e-5 of w
        assert np.abs(w - p.detach().numpy()).max() <= 2e-4 * 0.01
    assert (step == 4).all()


def test_adam_closed_forms():
    # first step from zero state: m = (1-b1) g, v = (1-b2) g^2, both bias corrections cancel,
    # so dw = -lr * g / (|g| + eps) = -lr * sign(g) up to rounding - a dropped correction, a
    # dropped sqrt or a wrong sign all fail this
    g = np.array([[3.0, -0.5, 1e-3, -2e-2]], np.float32)
    w0 = np.array([[1.0, 2.0, -3.0, 0.5]], np.float32)
    z1, z = np.zeros(1, np.float32), np.zeros_like(g)
    w1, step, m1, v1 = O.adam_rows(w0, z1, z, z, g, 0.01, 0.9, 0.999, 1e-12)
    assert np.allclose(w1 - w0, -0.01 * np.sign(g), rtol=1e-5) and step[0] == 1
    assert np.allclose(m1, 0.1 * g, rtol=1e-6) and np.allclose(v1, 0.001 * g * g, rtol=1e-5)
    # g = 0 from zero state: nothing moves but the step counter (0 / (0 + eps))
    w2, step2, m2, v2 = O.adam_rows(w0, z1, z, z, z, 0.01, 0.9, 0.999, 1e-8)
    assert np.array_equal(w2, w0) and step2[0] == 1 and not m2.any() and not v2.any()
    # second step with the same gradient: m and v follow the geometric sums, dw is again -lr*sign(g)
    w3, step3, m3, v3 = O.adam_rows(w1, step, m1, v1, g, 0.01, 0.9, 0.999, 1e-12)
    assert np.allclose(m3, (1 - 0.9 ** 2) * g, rtol=1e-6) and np.allclose(v3, (1 - 0.999 ** 2) * g * g, rtol=1e-5)
    assert np.allclose(w3 - w1, -0.01 * np.sign(g), rtol=2e-4) and step3[0] == 2


# ---- accumulator ----------------------------------------------------------------------------
def test_accumulator_flush_equals_combine_of_all_batches():
    rng = np.random.default_rng(12)
    acc = O.ColdGradAccumulatorModel(4)
    all_ids, all_g = [], []
    for _ in range(5):
        ids = _zipfish(rng, 400, 200)
        g = rng.standard_normal((400, 4)).astype(np.float32)
        u, s, c = O.combine_sequential(ids, g)
        acc.accumulate(u, s, c)
        all_ids.append(ids)
        all_g.append(g)
    ids, sums, cnts = acc.flush()
    u, s, c = O.combine_float64(np.concatenate(all_ids), np.concatenate(all_g))
    assert np.array_equal(ids, u) and np.array_equal(cnts, c)
    assert np.allclose(sums, s, rtol=1e-5, atol=1e-6)
    assert acc.flush()[0].size == 0          # emptied


# ---- C restatement vs numpy restatement -----------------------------------------------------
def test_c_oracle_agrees_with_numpy_oracle(oracle_c):
    C = oracle_c
    rng = np.random.default_rng(13)
    i64 = np.int64
    rng_part = np.array([0, 1000, 2500, 4000], i64)
    v = rng.integers(0, 4000, 777).astype(i64)
    out = np.empty_like(v)
    C.o_binary_search2(_p(v), _p(rng_part), ctypes.c_int64(4), _p(out), ctypes.c_int64(v.size))
    assert np.array_equal(out, O.upper_bound(rng_part, v))
    C.o_binary_search(_p(v), _p(rng_part), ctypes.c_int64(4), ctypes.c_int64(4), _p(out),
                      ctypes.c_int64(v.size))
    assert np.array_equal(out, O.owner_rank(v, rng_part, 4))
    vv = rng.integers(-100, 100, 50).astype(i64)
    o2 = np.empty_like(vv)
    C.o_reminder(_p(vv), ctypes.c_int64(7), _p(o2), ctypes.c_int64(vv.size))
    assert np.array_equal(o2, O.c_remainder(vv, 7))

    hot = np.sort(rng.choice(4000, 500, replace=False)).astype(i64)
    loc = np.empty_like(v)
    C.o_lookup_sorted(_p(v), ctypes.c_int64(v.size), _p(hot), ctypes.c_int64(hot.size), _p(loc))
    assert np.array_equal(loc, O.lookup_sorted(v, hot))

    table = rng.integers(0, 4, 4000).astype(np.int8)
    m = [np.empty(v.size, np.uint8) for _ in range(3)]
    C.o_split(_p(v), _p(table), ctypes.c_int64(v.size), _p(m[0]), _p(m[1]), _p(m[2]))
    for got, want in zip(m, O.split_masks(v, table)):
        assert np.array_equal(got.astype(bool), want)

    src, gpu_src, idx_map, q = _cache_case(rng)
    dst = np.empty((q.size, 8), np.float32)
    C.o_fetch_with_cache2(_p(src), _p(gpu_src), _p(q), _p(idx_map), _p(dst), ctypes.c_int64(q.size),
                          ctypes.c_int64(32))
    assert np.array_equal(dst, O.fetch_with_cache2(src, gpu_src, q, idx_map))
    C.o_fetch2(_p(src), _p(q), _p(dst), ctypes.c_int64(q.size), ctypes.c_int64(32))
    assert np.array_equal(dst, src[q])
    rows = rng.standard_normal((q.size, 8)).astype(np.float32)
    c_cpu, c_gpu = src.copy(), gpu_src.copy()
    C.o_set_with_cache(_p(rows), _p(c_cpu), _p(c_gpu), _p(q), _p(idx_map), ctypes.c_int64(q.size),
                       ctypes.c_int64(32))
    n_cpu, n_gpu = src.copy(), gpu_src.copy()
    O.set_with_cache(rows, n_cpu, n_gpu, q, idx_map)
    assert np.array_equal(c_cpu, n_cpu) and np.array_equal(c_gpu, n_gpu)

    idx = _zipfish(rng, 5000, 400)
    g = (rng.standard_normal((5000, 8)) * 1e-3).astype(np.float32)
    uids = np.empty(5000, i64); sums = np.empty((5000, 8), np.float32); cnts = np.empty(5000, i64)
    C.o_combine.restype = ctypes.c_int64
    U = C.o_combine(_p(idx), _p(g), ctypes.c_int64(5000), ctypes.c_int64(8), _p(uids), _p(sums), _p(cnts))
    nu, ns, nc = O.combine_sequential(idx, g)
    assert U == nu.size and np.array_equal(uids[:U], nu) and np.array_equal(cnts[:U], nc)
    assert np.array_equal(sums[:U], ns)

    n_rows = 4000
    cw = (rng.standard_normal((n_rows, 8)) * 0.01).astype(np.float32)
    cs = np.abs(rng.standard_normal((n_rows, 8))).astype(np.float32)
    hw, hs = cw[hot].copy(), cs[hot].copy()
    cw2, cs2, hw2, hs2 = cw.copy(), cs.copy(), hw.copy(), hs.copy()
    u = np.unique(v)
    gg = (rng.standard_normal((u.size, 8)) * 1e-3).astype(np.float32)
    C.o_adagrad(_p(u), _p(gg), ctypes.c_int64(u.size), ctypes.c_int64(8), _p(hot),
                ctypes.c_int64(hot.size), _p(hw), _p(hs), _p(cw), _p(cs), ctypes.c_float(0.01),
                ctypes.c_float(1e-10))
    O.sparse_adagrad_step(cw2, cs2, hw2, hs2, hot, u, gg, 0.01, 1e-10)
    for a, b in ((cw, cw2), (cs, cs2), (hw, hw2), (hs, hs2)):
        assert np.array_equal(a, b)


def test_torch_step_agrees_with_numpy_pieces():
    rng = np.random.default_rng(14)
    n_rows, dim = 5000, 8
    cw = (rng.standard_normal((n_rows, dim)) * 0.01).astype(np.float32)
    cs = np.zeros((n_rows, dim), np.float32)
    hot = np.sort(rng.choice(n_rows, 600, replace=False)).astype(np.int64)
    hw, hs = cw[hot].copy(), cs[hot].copy()
    q = _zipfish(rng, 3000, n_rows)
    g = (rng.standard_normal((3000, dim)) * 1e-3).astype(np.float32)
    t = [torch.from_numpy(x.copy()) for x in (cw, cs, hw, hs)]
    rows, uids, sums, cnts = O.torch_step(t[0], t[1], t[2], t[3], torch.from_numpy(hot),
                                          torch.from_numpy(q), torch.from_numpy(g), 0.01, 1e-10)
    assert np.array_equal(rows.numpy(), O.cached_fetch(cw, hw, q, hot))
    u, s, c = O.combine_sequential(q, g)
    assert np.array_equal(uids.numpy(), u) and np.array_equal(sums.numpy(), s)
    O.sparse_adagrad_step(cw, cs, hw, hs, hot, u, s, 0.01, 1e-10)
    for a, b in zip(t, (cw, cs, hw, hs)):
        assert np.allclose(a.numpy(), b, rtol=1e-5, atol=1e-9)


# ---- set-associative index cache ------------------------------------------------------------
def test_sacache_model_known_answers():
    # worked by hand from src/cache/cache_line.h: 2 lines of 8 entries, ids with id % 2 == 0 -> line 0
    m = O.SACacheIndexModel(16)
    assert m.lines == 2 and m.get_capacity() == 16
    # empty line: the LAST empty entry is taken (find_or_empty_entry keeps the last -1 it sees)
    assert m.add([0, 2, 4]).tolist() == [7, 6, 5]
    assert m.add([2]).tolist() == [6]                       # already present: same loc, no change
    assert m.add([1]).tolist() == [8 + 7]                   # line 1
    assert m.cudalookup([4, 6, 1, 3]).tolist() == [5, -1, 15, -1]
    assert m.add([6, 8, 10, 12, 14]).tolist() == [4, 3, 2, 1, 0]     # line 0 now full
    # nothing has been looked up yet: every age is 0 -> no victim -> -1
    assert m.add([16]).tolist() == [-1]
    # a hit ages every entry of the line by one and zeroes the hit
    assert m.lookup([0, 0]).tolist() == [7, 7]
    assert m.age[0].tolist() == [2, 2, 2, 2, 2, 2, 2, 0]
    # victim: the largest non-zero age, ties to the lowest entry -> entry 0 (id 14)
    assert m.add([16]).tolist() == [0]
    assert m.cudalookup([14, 16]).tolist() == [-1, 0]
    assert m.age[0].tolist() == [0, 2, 2, 2, 2, 2, 2, 0]
    assert m.add([18]).tolist() == [1]                      # next victim: entry 1 (id 12)
    m.reset([16, 99])                                       # absent ids are ignored
    assert m.cudalookup([16]).tolist() == [-1] and m.get_valid_entries_num() == 8
    assert m.add([20]).tolist() == [0]                      # the freed entry is reused
    ids, locs = m.getall(100)
    assert locs.tolist() == [0, 1, 2, 3, 4, 5, 6, 7, 15]
    assert ids.tolist() == [20, 18, 10, 8, 6, 4, 2, 0, 1]
    assert m.getall(3)[1].tolist() == [0, 1, 2]


@pytest.mark.parametrize("cache_size,id_range,seed", [(64, 400, 1), (1000, 3000, 2), (8, 50, 3)])
def test_sacache_model_matches_reference_cache_line(sacache_ref, cache_size, id_range, seed):
    # the model against the reference's own cache_line class on random operation sequences
    rng = np.random.default_rng(seed)
    m, r = O.SACacheIndexModel(cache_size), sacache_ref(cache_size)
    assert m.lines == r.lines
    for step in range(60):
        ids = rng.integers(0, id_range, int(rng.integers(1, 200))).astype(np.int64)
        op = step % 4
        if op == 0:
            assert np.array_equal(m.add(ids), r.add(ids))
        elif op == 1:
            assert np.array_equal(m.lookup(ids), r.lookup(ids))
        elif op == 2:
            assert np.array_equal(m.cudalookup(ids), r.cudalookup(ids))
            assert np.array_equal(m.add(np.unique(ids)), r.add(np.unique(ids)))
        else:
            m.reset(ids[:20]); r.reset(ids[:20])
        assert m.get_valid_entries_num() == r.get_valid_entries_num()
        a, b = m.getall(m.get_capacity()), r.getall(m.get_capacity())
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_cold_cache_server_model_against_per_id_bookkeeping():
    # The slot-array model against plain per-id bookkeeping in a setting without evictions
    # (at most 8 ids per line): what leaves at which flush, with which sum and count.
    rng = np.random.default_rng(31)
    n_ids, dim, lines = 400, 4, 64
    ids_all = np.arange(n_ids, dtype=np.int64)                   # id % 64: 6-7 ids per line
    hotness = rng.choice([0.0, 0.05, 0.3, 1.0, 5.0], n_ids).astype(np.float32)
    thr = np.minimum(np.ceil(1.0 / (np.float32(0.001) + hotness)), 100).astype(np.int64)
    m = O.ColdCacheServerModel(lines * 8, dim, hotness, cnt_threshold=3)
    assert np.array_equal(m.threshold.numpy(), thr)
    cached, pend, cnt, it = set(), {}, {}, {}
    for step in range(60):
        if step % 7 == 0:                                        # (re-)insert everything
            locs = m.update_cache(ids_all, rng.standard_normal((n_ids, dim)).astype(np.float32))
            assert (locs >= 0).all()
            for i in range(n_ids):
                cached.add(i); pend[i] = np.zeros(dim, np.float32); cnt[i] = 0; it.setdefault(i, 0)
        batch = rng.choice(n_ids, 90, replace=False).astype(np.int64)
        g = rng.standard_normal((batch.size, dim)).astype(np.float32)
        locs = m.accumulate_gradients_cold_remote(batch, g)
        for r, i in enumerate(batch.tolist()):
            assert (locs[r] >= 0) == (i in cached)
            if i in cached:
                pend[i] = (pend[i] + g[r]).astype(np.float32); cnt[i] += 1
        out_ids, out_g, out_c = m.staled_gradients_remote()
        want = {}
        for i in sorted(cached):
            if cnt[i] > 0:
                if it[i] >= thr[i] or cnt[i] >= 3:
                    want[i] = (pend[i].copy(), cnt[i])
                    pend[i][:] = 0; cnt[i] = 0; it[i] = 0
                else:
                    it[i] += 1
        cached -= set(want)
        assert sorted(out_ids.tolist()) == sorted(want)
        for r, i in enumerate(out_ids.tolist()):
            assert np.array_equal(out_g[r], want[i][0]) and out_c[r] == want[i][1]
        assert m.index.get_valid_entries_num() == len(cached)
    # the dense local part: same rule, ids = slot + part_start
    m = O.ColdCacheServerModel(64, dim, hotness, cnt_threshold=2, part_start=100, part_nnodes=50)
    lid = np.array([100, 149, 120], np.int64)
    lg = rng.standard_normal((3, dim)).astype(np.float32)
    m.accumulate_gradients_cold_local(lid, lg)
    m.accumulate_gradients_cold_local(lid[:1], lg[:1])
    out_ids, out_g, out_c = m.staled_gradients_local()
    due0 = [int(i) for i in (120, 149) if thr[i] <= 0]           # first flush: iter 0 >= thr never
    assert out_ids.tolist() == sorted([100] + due0)              # id 100 reached cnt_threshold
    assert np.array_equal(out_g[0], (lg[0] + lg[0]).astype(np.float32)) and out_c[0] == 2


def test_split_schedule_equals_the_unsplit_operators():
    """The class-by-class forms (python/EmbCache/dist_emb.py:174-211) against the one-kernel forms
    and against brute force: every row comes from the table its class says, lists are ascending
    and disjoint and cover the live prefix, entries beyond num_live are in neither list."""
    rng = np.random.default_rng(31)
    N, D, H, n = 3000, 5, 400, 2000
    cold = rng.standard_normal((N, D)).astype(np.float32)
    hot_ids = np.sort(rng.choice(N, H, replace=False)).astype(np.int64)
    hot = cold[hot_ids] + 100.0      # hot copies differ from the cold copies: the source shows
    q = rng.integers(0, N, n).astype(np.int64)
    loc, hot_pos, cold_pos = O.lookup_split(q, hot_ids)
    member = {int(v): k for k, v in enumerate(hot_ids)}
    assert [member.get(int(v), -1) for v in q] == loc.tolist()
    assert sorted(hot_pos.tolist() + cold_pos.tolist()) == list(range(n))
    assert np.all(np.diff(hot_pos) > 0) and np.all(np.diff(cold_pos) > 0)
    assert all(int(q[p]) in member for p in hot_pos) and not any(int(q[p]) in member for p in cold_pos)
    out = O.fetch_split(cold, hot, q, hot_ids)
    assert np.array_equal(out, O.cached_fetch(cold, hot, q, hot_ids))
    assert np.array_equal(out[hot_pos], hot[loc[hot_pos]]) and np.array_equal(out[cold_pos], cold[q[cold_pos]])
    # num_live
    loc2, hp2, cp2 = O.lookup_split(q, hot_ids, num_live=700)
    assert hp2.tolist() == [p for p in hot_pos if p < 700] and cp2.tolist() == [p for p in cold_pos if p < 700]
    assert O.lookup_split(q, hot_ids, num_live=-1)[1].size == 0
    # a partial count leaves the other positions alone
    out3 = np.full((n, D), -7.0, np.float32)
    O.fetch_listed(cold, q, cold_pos, 10, out3)
    assert np.array_equal(out3[cold_pos[:10]], cold[q[cold_pos[:10]]])
    rest = np.ones(n, bool); rest[cold_pos[:10]] = False
    assert np.all(out3[rest] == -7.0)
    # set_listed is the inverse scatter
    uq = rng.permutation(N)[:n].astype(np.int64)
    l3, hp3, cp3 = O.lookup_split(uq, hot_ids)
    src = rng.standard_normal((n, D)).astype(np.float32)
    c_a, h_a = cold.copy(), hot.copy()
    O.set_listed(src, h_a, l3, hp3, hp3.size)
    O.set_listed(src, c_a, uq, cp3, cp3.size)
    c_b, h_b = cold.copy(), hot.copy()
    O.cached_set(src, c_b, h_b, uq, hot_ids)
    assert np.array_equal(c_a, c_b) and np.array_equal(h_a, h_b)
    # the update, class by class == the fused form; rows of no class do not move
    g = (rng.standard_normal((n, D)) * 1e-3).astype(np.float32)
    s0 = np.abs(rng.standard_normal((N, D))).astype(np.float32)
    a = [cold.copy(), s0.copy(), hot.copy(), s0[hot_ids].copy()]
    b = [x.copy() for x in a]
    O.sparse_adagrad_step(a[0], a[1], a[2], a[3], hot_ids, uq[:1500], g[:1500], 0.01, 1e-10)
    O.sparse_adagrad_step_split(b[0], b[1], b[2], b[3], hot_ids, uq, g, 0.01, 1e-10, num_live=1500)
    for x, y in zip(a, b):
        assert np.array_equal(x, y)


def test_keyed_step_equals_combine_then_update_on_the_ids():
    """Sorting by (class, id-or-slot) instead of by id changes the order of the distinct rows and
    nothing else: same sums per id (same occurrence order inside a run), same tables afterwards."""
    rng = np.random.default_rng(77)
    N, D, H, n = 5000, 6, 700, 9000
    kb = 13
    cold = rng.standard_normal((N, D)).astype(np.float32)
    hot_ids = np.sort(rng.choice(N, H, replace=False)).astype(np.int64)
    q = np.minimum(rng.pareto(0.8, n).astype(np.int64) * 37 % N, N - 1)
    g = (rng.standard_normal((n, D)) * 1e-2).astype(np.float32)
    a = [cold.copy(), np.zeros((N, D), np.float32), cold[hot_ids] + 1, np.zeros((H, D), np.float32)]
    b = [x.copy() for x in a]
    for _ in range(2):
        wu, ws, wc = O.combine_sequential(q, g)
        O.sparse_adagrad_step(a[0], a[1], a[2], a[3], hot_ids, wu, ws, 0.01, 1e-10)
        ukeys, sums, cnts, split = O.keyed_step(b[0], b[1], b[2], b[3], hot_ids, q, g, 0.01, 1e-10, kb)
        # the keyed rows are the id rows in another order
        ids = np.where(ukeys >= (1 << kb), hot_ids[np.maximum(ukeys - (1 << kb), 0) % H], ukeys)
        order = np.argsort(ids, kind="stable")
        assert np.array_equal(ids[order], wu) and np.array_equal(sums[order], ws) and np.array_equal(cnts[order], wc)
        assert np.all(np.diff(ukeys) > 0) and np.all(ukeys[:split] < (1 << kb)) and np.all(ukeys[split:] >= (1 << kb))
        assert not np.isin(ukeys[:split], hot_ids).any()
    for x, y in zip(a, b):
        assert np.array_equal(x, y)
    # with the rows a forward pass fetched (= the table rows) nothing changes
    c = [x.copy() for x in b]
    O.keyed_step(b[0], b[1], b[2], b[3], hot_ids, q, g, 0.01, 1e-10, kb)
    O.keyed_step(c[0], c[1], c[2], c[3], hot_ids, q, g, 0.01, 1e-10, kb,
                 fetched_rows=O.cached_fetch(c[0], c[2], q, hot_ids))
    for x, y in zip(b, c):
        assert np.array_equal(x, y)


def test_keyed_step_adam_equals_combine_then_adam_on_the_ids():
    """keyed_step_adam (class-ordered keys, per-class tables) must give what the reference's flow
    gives on the ids: unique + index_add (only_unique_grads, python/EmbCache/sparse_optim.py:132-139)
    and then adam_rows on the gathered rows of each distinct id (:590-685), whichever table holds
    the row.  Also adam_listed class by class."""
    rng = np.random.default_rng(5)
    N, D, H, n = 400, 8, 60, 1500
    hot_ids = np.sort(rng.choice(N, H, replace=False)).astype(np.int64)
    w0 = rng.standard_normal((N, D)).astype(np.float32)
    q = rng.integers(0, N, n).astype(np.int64)
    kb = 9
    cold = (w0.copy(), np.zeros(N, np.float32), np.zeros_like(w0), np.zeros_like(w0))
    hot = tuple(x[hot_ids].copy() for x in cold)
    full = tuple(x.copy() for x in cold)                  # one table, no cache: the plain flow
    lcold = tuple(x.copy() for x in cold)
    lhot = tuple(x.copy() for x in hot)
    for it in range(3):
        grad = rng.standard_normal((n, D)).astype(np.float32)
        ukeys, sums, cnts, split = O.keyed_step_adam(cold, hot, hot_ids, q, grad, 0.01, 0.9, 0.999, 1e-8, kb)
        uids, usum, ucnt = O.combine_sequential(q, grad)
        res = O.adam_rows(full[0][uids], full[1][uids], full[2][uids], full[3][uids], usum,
                          0.01, 0.9, 0.999, 1e-8)
        for k in range(4):
            full[k][uids] = res[k]
        # the listed form on the distinct ids
        loc, hot_pos, cold_pos = O.lookup_split(uids, hot_ids)
        O.adam_listed(loc, usum, hot_pos, hot_pos.size, *lhot, 0.01, 0.9, 0.999, 1e-8)
        O.adam_listed(uids, usum, cold_pos, cold_pos.size, *lcold, 0.01, 0.9, 0.999, 1e-8)
        assert split == (O.lookup_sorted(uids, hot_ids) < 0).sum()
    is_hot = np.zeros(N, bool); is_hot[hot_ids] = True
    for k in range(4):
        merged = cold[k].copy(); merged[hot_ids] = hot[k]
        assert np.array_equal(merged, full[k])
        lm = lcold[k].copy(); lm[hot_ids] = lhot[k]
        assert np.array_equal(lm, full[k])
        # the cold table's rows of hot ids were never touched
        init = (w0, np.zeros(N, np.float32), np.zeros_like(w0), np.zeros_like(w0))[k]
        assert np.array_equal(cold[k][is_hot], init[is_hot])
