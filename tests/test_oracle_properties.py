"""Property tests of the CPU oracle on generated inputs (hypothesis): the invariants the
mathematics fixes, whatever the data.  No GPU."""
import bisect

import numpy as np
import torch
from hypothesis import given, settings, strategies as st

from oracle import hades_oracle as O

SMALL = settings(max_examples=60, deadline=None)
ids_lists = st.lists(st.integers(min_value=0, max_value=40), min_size=0, max_size=60)


@SMALL
@given(st.lists(st.integers(-50, 50), max_size=30), st.lists(st.integers(-60, 60), max_size=40))
def test_upper_bound_is_bisect_right(rng_vals, queries):
    r = np.array(sorted(rng_vals), dtype=np.int64)
    q = np.array(queries, dtype=np.int64)
    want = np.array([bisect.bisect_right(r.tolist(), x) for x in queries], dtype=np.int64)
    assert np.array_equal(O.upper_bound(r, q), want)


@SMALL
@given(st.sets(st.integers(0, 60), max_size=25), st.lists(st.integers(-3, 63), max_size=40))
def test_lookup_sorted_is_membership_with_rank(hot, queries):
    hot = np.array(sorted(hot), dtype=np.int64)
    q = np.array(queries, dtype=np.int64)
    loc = O.lookup_sorted(q, hot)
    for x, l in zip(queries, loc.tolist()):
        assert (l >= 0) == (x in set(hot.tolist()))
        if l >= 0:
            assert hot[l] == x


@SMALL
@given(ids_lists, st.integers(1, 5))
def test_combine_invariants(ids, dim):
    idx = np.array(ids, dtype=np.int64)
    rng = np.random.default_rng(len(ids) * 7 + dim)
    grad = rng.standard_normal((idx.size, dim)).astype(np.float32)
    uids, sums, cnts = O.combine_sequential(idx, grad)
    assert np.array_equal(uids, np.unique(idx)) and int(cnts.sum()) == idx.size
    assert np.all(np.diff(uids) > 0)
    for k, u in enumerate(uids.tolist()):
        rows = grad[idx == u]
        acc = np.zeros(dim, np.float32)
        for r in rows:                       # the same left-to-right float32 chain
            acc = (acc + r).astype(np.float32)
        assert np.array_equal(sums[k], acc) and cnts[k] == rows.shape[0]
    if idx.size:
        tu, ts, tc = O.only_unique_grads(torch.from_numpy(idx), torch.from_numpy(grad))
        assert np.array_equal(tu.numpy(), uids) and np.array_equal(tc.numpy(), cnts)
        assert np.array_equal(ts.numpy(), sums)
    # any permutation of the batch gives the same ids and counts, and the same sums to rounding
    perm = rng.permutation(idx.size)
    u2, s2, c2 = O.combine_sequential(idx[perm], grad[perm])
    assert np.array_equal(u2, uids) and np.array_equal(c2, cnts)
    assert np.allclose(s2, sums, rtol=1e-5, atol=1e-5)


@SMALL
@given(ids_lists, st.integers(1, 6), st.booleans())
def test_bucket_by_owner_is_a_stable_partition(ids, local, ranged):
    idx = np.array(ids, dtype=np.int64)
    rp = np.array([0, 15, 41], np.int64) if ranged else None
    G = (2 if ranged else 1) * local
    b_ids, _, _, sizes, perm = O.bucket_by_owner(idx, rp, local, G)
    assert sorted(perm.tolist()) == list(range(idx.size)) and int(sizes.sum()) == idx.size
    owner = O.owner_rank(idx, rp, local) if ranged else O.c_remainder(idx, local)
    assert np.array_equal(b_ids, idx[perm])
    assert np.all(np.diff(owner[perm]) >= 0)                       # grouped by owner
    start = 0
    for g in range(G):
        seg = perm[start:start + int(sizes[g])]
        assert np.all(owner[seg] == g) and np.all(np.diff(seg) > 0)   # input order inside a bucket
        start += int(sizes[g])


ops_strategy = st.lists(
    st.tuples(st.sampled_from(["add", "lookup", "reset", "cudalookup"]),
              st.lists(st.integers(0, 70), min_size=0, max_size=25)),
    min_size=1, max_size=25)


@SMALL
@given(st.integers(1, 40), ops_strategy)
def test_index_cache_model_invariants(cache_size, program):
    m = O.SACacheIndexModel(cache_size)
    for op, ids in program:
        ids = np.array(ids, dtype=np.int64)
        if op == "add":
            locs = m.add(ids)
            for x, l in zip(ids.tolist(), locs.tolist()):
                if l >= 0:                                   # a loc handed out names the id's own line
                    assert l // 8 == x % m.lines
            # what add reported present is found by a lookup that changes nothing - unless a later
            # id of the same batch took the entry over
            found = m.cudalookup(ids)
            for x, l, f in zip(ids.tolist(), locs.tolist(), found.tolist()):
                assert f == -1 or m.ids.reshape(-1)[f] == x
        elif op == "lookup":
            before = m.ids.copy()
            a = m.lookup(ids)
            assert np.array_equal(m.ids, before)             # lookups never move ids
            assert np.array_equal(a, m.cudalookup(ids))
        elif op == "reset":
            m.reset(ids)
            assert np.all(m.cudalookup(ids) == -1)
        else:
            before_ids, before_age = m.ids.copy(), m.age.copy()
            m.cudalookup(ids)
            assert np.array_equal(m.ids, before_ids) and np.array_equal(m.age, before_age)
        flat = m.ids.reshape(-1)
        live = flat[flat != -1]
        assert live.size == np.unique(live).size             # an id is cached at most once
        assert m.get_valid_entries_num() == live.size <= m.get_capacity()
        assert np.all(m.age >= 0)      # (a hit ages the empty entries of its line too, as access_loc does)
