"""GPU parity: every operator of the C-ABI library against the CPU oracle on the same seeded
inputs.  Integer, index and payload results must be bit-exact; float32 sums and updates are
bit-exact in the deterministic modes and within the stated tolerance otherwise."""
import numpy as np
import pytest
import torch

from oracle import hades_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib(cuda_device):
    import hades_amd.EmbCacheLib as E
    from hades_amd import ops
    return E, ops


def dev(a, device="cuda"):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def zipfish(rng, n, n_ids):
    return np.minimum((rng.pareto(0.9, n)).astype(np.int64), n_ids - 1)


NP_F = {torch.float32: np.float32, torch.float64: np.float64}
NP_I = {torch.int32: np.int32, torch.int64: np.int64}


# ---- cudaFetch* / cudaSet* / cudaCombine: the reference's test recipes --------------------
@pytest.mark.parametrize("dim", [1, 3, 7, 64, 100, 128, 260])
@pytest.mark.parametrize("fdt,idt", [(torch.float32, torch.int64), (torch.float64, torch.int32)])
@pytest.mark.parametrize("host_cold", [False, True])
def test_fetch_and_set_with_cache(lib, dim, fdt, idt, host_cold):
    E, _ = lib
    rng = np.random.default_rng(100 + dim)
    n_rows, n_cached, n_q = 5000, 2000, 1537
    shape = (n_rows,) if dim == 1 else (n_rows, dim)
    src = rng.standard_normal(shape).astype(NP_F[fdt])
    cached_idx = rng.permutation(n_rows)[:n_cached]
    idx_map = O.dense_index_map(n_rows, cached_idx, NP_I[idt])
    gpu_src_np = src[cached_idx].copy()
    q = rng.permutation(n_rows)[:n_q].astype(NP_I[idt])

    if host_cold:
        cpu_src = torch.empty(shape, dtype=fdt, pin_memory=True)
        cpu_src.copy_(torch.from_numpy(src))
        E.cudaPin(cpu_src)          # already page-locked: a no-op, as for the reference after pinning
    else:
        cpu_src = dev(src)
    gpu_src, d_map, d_q = dev(gpu_src_np), dev(idx_map), dev(q)
    dst = torch.zeros((n_q,) + shape[1:], dtype=fdt, device="cuda")

    # test/test_cached_fetch.py:52-60 / :66-74 (and _1D)
    E.cudaFetchWithCache2(cpu_src, gpu_src, d_q, d_map, dst)
    torch.cuda.synchronize()
    assert np.array_equal(dst.cpu().numpy(), O.fetch_with_cache2(src, gpu_src_np, q, idx_map))
    assert np.array_equal(dst.cpu().numpy(), src[q])
    dst.zero_()
    E.cudaFetch2(cpu_src, d_q, dst)
    torch.cuda.synchronize()
    assert np.array_equal(dst.cpu().numpy(), O.fetch2(src, q))

    # test/test_cached_set.py:50-58 / :64-72
    rows = rng.standard_normal((n_q,) + shape[1:]).astype(NP_F[fdt])
    want_cpu, want_gpu = src.copy(), gpu_src_np.copy()
    O.set_with_cache(rows, want_cpu, want_gpu, q, idx_map)
    E.cudaSetWithCache(dev(rows), cpu_src, gpu_src, d_q, d_map)
    torch.cuda.synchronize()
    assert np.array_equal(cpu_src.cpu().numpy(), want_cpu)
    assert np.array_equal(gpu_src.cpu().numpy(), want_gpu)
    want = want_cpu.copy()
    O.set_rows(rows, want, q)
    E.cudaSet(dev(rows), cpu_src, d_q)
    torch.cuda.synchronize()
    assert np.array_equal(cpu_src.cpu().numpy(), want)


@pytest.mark.parametrize("dim", [4, 128, 33])
def test_fetch_dst_indexed_and_combine_scatter(lib, dim):
    E, _ = lib
    rng = np.random.default_rng(200 + dim)
    src = rng.standard_normal((4000, dim)).astype(np.float32)
    dst = rng.standard_normal((900, dim)).astype(np.float32)
    si = rng.permutation(4000)[:700].astype(np.int64)
    di = rng.permutation(900)[:700].astype(np.int64)
    d_dst = dev(dst)
    E.cudaFetch(dev(src), dev(si), d_dst, dev(di))                 # test/test_fetch.py:31
    torch.cuda.synchronize()
    assert np.array_equal(d_dst.cpu().numpy(), O.fetch(src, si, dst.copy(), di))
    big = np.zeros((4000, dim), np.float32)
    d_big = dev(big)
    rows = rng.standard_normal((700, dim)).astype(np.float32)
    E.cudaCombine(dev(rows), d_big, dev(si))                        # test/test_combine.py:33
    torch.cuda.synchronize()
    assert np.array_equal(d_big.cpu().numpy(), O.set_rows(rows, big.copy(), si))


def test_mover_unaligned_views_and_empty(lib):
    E, _ = lib
    rng = np.random.default_rng(3)
    base = torch.from_numpy(rng.standard_normal(4 * 1000 + 1).astype(np.float32)).cuda()
    src = base[1:].view(1000, 4)            # 4-byte aligned only: takes the narrow copy path
    assert src.data_ptr() % 16 != 0
    q = rng.integers(0, 1000, 333).astype(np.int64)
    dst = torch.empty((333, 4), device="cuda")
    E.cudaFetch2(src, dev(q), dst)
    torch.cuda.synchronize()
    assert torch.equal(dst.cpu(), src.cpu()[torch.from_numpy(q)])
    empty = torch.empty(0, dtype=torch.int64, device="cuda")
    E.cudaFetch2(src, empty, torch.empty((0, 4), device="cuda"))
    E.cudaSet(torch.empty((0, 4), device="cuda"), src, empty)
    torch.cuda.synchronize()


def test_shim_rejects_bad_arguments(lib):
    E, _ = lib
    a = torch.zeros((10, 4), device="cuda")
    i = torch.zeros(3, dtype=torch.int64, device="cuda")
    with pytest.raises(RuntimeError):
        E.cudaFetch(a, i, torch.zeros((10, 5), device="cuda"), i)       # CHECK(src.size(1) == dst.size(1))
    with pytest.raises(RuntimeError):
        E.cudaFetch(a, i, a, torch.zeros(4, dtype=torch.int64, device="cuda"))
    with pytest.raises(RuntimeError):
        E.cudaFetch2(a.half(), i, a.half())                              # float or double only
    with pytest.raises(RuntimeError):
        E.cudaFetch2(a, i.to(torch.int16), a)                            # int32 or int64 only
    with pytest.raises(RuntimeError):
        E.cudaFetch2(torch.zeros((10, 4)), i, a)                         # pageable host memory
    with pytest.raises(RuntimeError):
        E.cudaFetch2(a.t(), i, a)                                        # not contiguous


# ---- routing ----------------------------------------------------------------------------
@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
def test_routing_ops(lib, idt):
    E, _ = lib
    rng = np.random.default_rng(4)
    v = rng.integers(0, 3_000_000, 10_001).astype(NP_I[idt])
    rp = np.array([0, 1_500_000, 3_000_000], NP_I[idt])
    assert np.array_equal(E.cudaReminder(dev(v), 4).cpu().numpy(), O.c_remainder(v, 4))
    owner = E.cudaBinarySearch(dev(v), dev(rp), 4)
    assert owner.dtype == idt
    assert np.array_equal(owner.cpu().numpy(), O.owner_rank(v, rp, 4))
    # split sizes (test/test_binarysearch2.py:19-27, python/EmbCache/sparse_optim.py:43-54)
    value, _ = torch.sort(owner)
    ranges = torch.arange(8, device="cuda", dtype=idt)
    splits = E.cudaBinarySearch2(ranges, value)
    assert np.array_equal(splits.cpu().numpy(), O.upper_bound(np.sort(O.owner_rank(v, rp, 4)), np.arange(8, dtype=NP_I[idt])))
    splits[1:] = splits[1:] - splits[:-1].clone()
    assert np.array_equal(splits.cpu().numpy().astype(np.int64), O.split_sizes(np.sort(O.owner_rank(v, rp, 4)), 8))
    # negative values: C remainder
    neg = np.array([-7, 7, -1, 0], NP_I[idt])
    assert np.array_equal(E.cudaReminder(dev(neg), 4).cpu().numpy(), O.c_remainder(neg, 4))
    # empty range / empty input
    assert E.cudaBinarySearch2(dev(v), torch.empty(0, dtype=idt, device="cuda")).sum().item() == 0
    assert E.cudaReminder(torch.empty(0, dtype=idt, device="cuda"), 4).numel() == 0


# ---- pre-exchange bucketing (swap_gradients before its all-to-all) ---------------------------
@pytest.mark.parametrize("n,num_part,local,dim,fdt", [
    (10_001, 2, 4, 16, torch.float32),     # partition range, 8 owners
    (50_000, 1, 8, 128, torch.float32),    # remainder only (partition_range=None)
    (7_777, 5, 64, 3, torch.float64),      # 320 owners: two sort passes
    (1, 1, 1, 4, torch.float32),           # one row, one owner
    (300_000, 4, 8, 8, torch.float32),     # several tiles per group
])
def test_bucket_by_owner(lib, n, num_part, local, dim, fdt):
    _, ops = lib
    rng = np.random.default_rng(n + local)
    n_rows = 3_000_000
    ids = rng.integers(0, n_rows, n).astype(np.int64)
    grad = rng.standard_normal((n, dim)).astype(NP_F[fdt])
    cnt = rng.integers(1, 100, n).astype(np.int64)
    ranged = num_part > 1
    rp = np.array([i * n_rows // num_part for i in range(num_part + 1)], np.int64) if ranged else None
    G = num_part * local
    want = O.bucket_by_owner(ids, rp, local, G, grad, cnt)
    got = ops.bucket_by_owner(dev(ids), dev(grad), dev(cnt), dev(rp) if ranged else None, local, G,
                              return_perm=True)
    for w, g in zip(want, got):
        assert w.dtype == g.cpu().numpy().dtype and np.array_equal(w, g.cpu().numpy())
    # ids only
    ids_out, g_out, c_out, sizes = ops.bucket_by_owner(dev(ids), None, None,
                                                       dev(rp) if ranged else None, local, G)
    assert g_out is None and c_out is None
    assert np.array_equal(ids_out.cpu().numpy(), want[0]) and np.array_equal(sizes.cpu().numpy(), want[3])


def test_bucket_by_owner_reference_names_and_empty(lib):
    _, ops = lib
    from hades_amd import sparse_optim
    rng = np.random.default_rng(77)
    ids = rng.integers(0, 1000, 4096).astype(np.int64)
    grad = rng.standard_normal((ids.size, 8)).astype(np.float32)
    rp = np.array([0, 400, 1000], np.int64)
    b_ids, b_grad, b_cnt, splits = sparse_optim.bucket_gradients(dev(ids), dev(grad), dev(rp), 2, 4)
    want = O.bucket_by_owner(ids, rp, 4, 8, grad)
    assert b_cnt is None
    assert np.array_equal(b_ids.cpu().numpy(), want[0]) and np.array_equal(b_grad.cpu().numpy(), want[1])
    assert splits.tolist() == want[3].tolist() and sum(splits.tolist()) == ids.size
    # empty batch: all sizes zero (python/EmbCache/sparse_optim.py:54-62)
    e_ids, e_grad, _, e_splits = ops.bucket_by_owner(
        torch.empty(0, dtype=torch.int64, device="cuda"),
        torch.empty((0, 8), dtype=torch.float32, device="cuda"), None, None, 4, 4)
    assert e_ids.numel() == 0 and e_grad.shape == (0, 8) and e_splits.tolist() == [0, 0, 0, 0]
    # an owner outside [0, num_owners) makes every split size -1
    bad = ops.bucket_by_owner(dev(np.array([5, -3, 7], np.int64)), None, None, None, 4, 4)
    assert bad[3].tolist() == [-1, -1, -1, -1]
    big = rng.integers(0, 1000, 20_000).astype(np.int64)
    big[12_345] = 1000                                  # beyond the last range: owner 8 of 8
    bad = ops.bucket_by_owner(dev(big), None, None, dev(rp), 4, 8)
    assert bad[3].tolist() == [-1] * 8


# ---- set-associative index cache (EmbCacheLib.IndexCache) ----------------------------------
def _same_cache_state(ic, model_or_ref):
    cap = ic.get_capacity()
    ids, locs, num = ic.getall_padded(cap)
    k = int(num.item())
    want_ids, want_locs = model_or_ref.getall(cap)
    assert k == want_ids.size == model_or_ref.get_valid_entries_num() == ic.get_valid_entries_num()
    assert np.array_equal(ids[:k].cpu().numpy(), want_ids)
    assert np.array_equal(locs[:k].cpu().numpy(), want_locs)


@pytest.mark.parametrize("cache_size,id_range,seed", [(64, 400, 1), (1000, 3000, 2), (8, 50, 3)])
def test_index_cache_random_sequences_vs_model(lib, cache_size, id_range, seed):
    import hades_amd.EmbCacheLib as E
    rng = np.random.default_rng(seed)
    ic, m = E.IndexCache(cache_size, "unused", True), O.SACacheIndexModel(cache_size)
    assert ic.get_capacity() == m.get_capacity() and ic.get_size() == m.get_capacity()
    assert ic.get_space() == m.lines * 96
    for step in range(40):
        ids = rng.integers(0, id_range, int(rng.integers(1, 300))).astype(np.int64)
        op = step % 4
        if op == 0:
            assert np.array_equal(ic.add(dev(ids)).cpu().numpy(), m.add(ids))
        elif op == 1:
            assert np.array_equal(ic.lookup(dev(ids)).cpu().numpy(), m.lookup(ids))
        elif op == 2:
            assert np.array_equal(ic.cudalookup(dev(ids)).cpu().numpy(), m.cudalookup(ids))
            u = np.unique(ids)
            assert np.array_equal(ic.add(dev(u)).cpu().numpy(), m.add(u))
        else:
            ic.reset(dev(ids[:20])); m.reset(ids[:20])
        _same_cache_state(ic, m)
        assert np.array_equal(ic.line_age.cpu().numpy().reshape(-1, 8), m.age)


def test_index_cache_known_answers_and_edges(lib):
    from hades_amd.index_cache import LocalCache
    t = lambda *v: torch.tensor(v, dtype=torch.int64, device="cuda")
    c = LocalCache("unused", 16, True)
    assert c.get_num_entries() == 16
    assert c.add(t(0, 2, 4)).tolist() == [7, 6, 5]           # last empty entry first
    assert c.add(t(2)).tolist() == [6]
    assert c.add(t(6, 8, 10, 12, 14)).tolist() == [4, 3, 2, 1, 0]
    assert c.add(t(16)).tolist() == [-1]                     # full line, all ages 0: no victim
    assert c.lookup(t(0, 0)).tolist() == [7, 7]
    assert c.add(t(16)).tolist() == [0]                      # oldest entry, lowest index on ties
    assert c.cudalookup(t(14, 16, 1, -5, -1)).tolist() == [-1, 0, -1, -1, -1]
    assert c.add(t(-5, 18)).tolist() == [-1, 1]              # negative ids are never cached
    c.reset(t(16, 99, -1))
    assert c.cudalookup(t(16)).tolist() == [-1]
    ids, locs = c._idx_cache.getall(3)
    assert locs.tolist() == [1, 2, 3] and ids.tolist() == [18, 10, 8]
    ids, locs = c._idx_cache.getall(12)                      # padded like the reference: 0 / -1
    assert locs.tolist()[7:] == [-1] * 5 and ids.tolist()[7:] == [0] * 5
    assert c.add(torch.empty(0, dtype=torch.int64, device="cuda")).numel() == 0


@pytest.mark.parametrize("cache_size,id_range,batch", [(100_000, 1_000_000, 60_000),
                                                       (4096, 50_000, 200_000)])
def test_index_cache_large_vs_reference_cache_line(lib, sacache_ref, cache_size, id_range, batch):
    # the reference's own cache_line class (oracle/_ref) on batches far larger than a line:
    # long per-line sequences, evictions, re-insertions
    import hades_amd.EmbCacheLib as E
    rng = np.random.default_rng(cache_size)
    ic, r = E.IndexCache(cache_size, "unused", True), sacache_ref(cache_size)
    for step in range(6):
        ids = rng.integers(0, id_range, batch).astype(np.int64)
        assert np.array_equal(ic.add(dev(ids)).cpu().numpy(), r.add(ids))
        probe = rng.integers(0, id_range, batch).astype(np.int64)
        assert np.array_equal(ic.cudalookup(dev(probe)).cpu().numpy(), r.cudalookup(probe))
        assert np.array_equal(ic.lookup(dev(probe)).cpu().numpy(), r.lookup(probe))
        gone = np.unique(ids[: batch // 10])                  # reset takes distinct ids
        ic.reset(dev(gone)); r.reset(gone)
        _same_cache_state(ic, r)


def test_index_cache_generated_programs_vs_model(lib):
    """Generated operation sequences (hypothesis) on tiny caches, where lines fill up, evict and
    are reset all the time: locs, line contents and ages after every operation."""
    from hypothesis import HealthCheck, given, settings, strategies as st
    import hades_amd.EmbCacheLib as E
    program = st.lists(st.tuples(st.sampled_from(["add", "lookup", "reset", "cudalookup"]),
                                 st.lists(st.integers(-2, 70), min_size=0, max_size=25)),
                       min_size=1, max_size=20)

    @settings(max_examples=40, deadline=None, suppress_health_check=list(HealthCheck))
    @given(st.integers(1, 40), program)
    def run(cache_size, prog):
        ic, m = E.IndexCache(cache_size, "unused", True), O.SACacheIndexModel(cache_size)
        for op, ids in prog:
            ids = np.array(ids, dtype=np.int64)
            ok = ids[ids >= 0]                      # the model, like the reference, takes ids >= 0
            if op == "reset":
                ic.reset(dev(ids)); m.reset(ok)
            else:
                got = getattr(ic, op)(dev(ids)).cpu().numpy()
                want = np.full(ids.shape, -1, np.int64)
                want[ids >= 0] = getattr(m, op)(ok)
                assert np.array_equal(got, want), (op, ids.tolist())
            assert np.array_equal(ic.line_ids.cpu().numpy().reshape(-1, 8), m.ids)
            assert np.array_equal(ic.line_age.cpu().numpy().reshape(-1, 8), m.age)

    run()


def test_index_cache_reference_recipes_at_their_sizes(lib, sacache_ref):
    """The reference's own scripts at their sizes, with assertions where they print:
    test/test_lookup.py (a 4 M-entry cache, ten adds of 2 M random ids, then ten 400 K-id lookups whose
    host and device results must agree, :8-35) and test/test_single_cache.py (ten rounds of add 200 K /
    lookup 200 K / reset 20 K, then get_valid_entries_num and getall, :13-40)."""
    import hades_amd.EmbCacheLib as E
    g = torch.Generator().manual_seed(42)
    size = 4_000_000
    ic, r = E.IndexCache(size, "test_cache", True), sacache_ref(size)
    assert ic.get_valid_entries_num() == 0
    for i in range(10):                                                   # test_lookup.py:12-14
        index = torch.randint(0, size, (2_000_000,), generator=g)
        assert np.array_equal(ic.add(index.cuda()).cpu().numpy(), r.add(index.numpy()))
    for i in range(10):                                                   # test_lookup.py:17-35
        index = torch.randint(0, size, (400_000,), generator=g)
        out1 = ic.lookup(index.cuda())
        out2 = ic.cudalookup(index.cuda())
        assert torch.equal(out1, out2)                                    # :34
        assert np.array_equal(out1.cpu().numpy(), r.lookup(index.numpy()))
    ic, r = E.IndexCache(size, "test_cache", True), sacache_ref(size)
    for i in range(10):                                                   # test_single_cache.py:13-34
        index = torch.randint(0, size, (200_000,), generator=g)
        assert np.array_equal(ic.add(index.cuda()).cpu().numpy(), r.add(index.numpy()))
        index = torch.randint(0, size, (200_000,), generator=g)
        assert np.array_equal(ic.lookup(index.cuda()).cpu().numpy(), r.lookup(index.numpy()))
        index = torch.unique(torch.randint(0, size, (20_000,), generator=g))
        ic.reset(index.cuda()); r.reset(index.numpy())
    assert ic.get_valid_entries_num() == r.get_valid_entries_num() > 0    # :36
    a, b = ic.getall(size)                                                # :37-39
    want_a, want_b = r.getall(size)
    k = want_a.size
    assert np.array_equal(a[:k].cpu().numpy(), want_a) and np.array_equal(b[:k].cpu().numpy(), want_b)
    assert int((b[k:] != -1).sum()) == 0 and int(a[k:].abs().sum()) == 0


# ---- cold-data cache: the server's gradient path with its staleness rule -------------------
def _cold_state_equal(c, m):
    assert np.array_equal(c.emb_cache_buff.cpu().numpy(), m.emb.numpy())
    assert np.array_equal(c.grad_cache_buff.cpu().numpy(), m.grad.numpy())
    assert np.array_equal(c.grad_cnt_cache_buff.cpu().numpy(), m.cnt.numpy())
    assert np.array_equal(c.grad_iter_count.cpu().numpy(), m.iter.numpy())
    live = m.cnt.numpy() > 0                       # ids and thresholds matter where gradients wait
    assert np.array_equal(c.grad_idx_cache_buff.cpu().numpy()[live], m.idx.numpy()[live])
    assert np.array_equal(c.grad_iter_threshold.cpu().numpy()[live], m.iter_thr.numpy()[live])
    assert np.array_equal(c.index.line_ids.cpu().numpy().reshape(-1, 8), m.index.ids)
    assert np.array_equal(c.index.line_age.cpu().numpy().reshape(-1, 8), m.index.age)


@pytest.mark.parametrize("cache_size,n_ids,dim,seed", [(256, 600, 8, 1), (64, 2000, 128, 2),
                                                       (1024, 1500, 3, 3)])
def test_cold_data_cache_vs_server_model(lib, cache_size, n_ids, dim, seed):
    from hades_amd.cold_cache import ColdDataCache
    rng = np.random.default_rng(seed)
    hotness = rng.choice([0.0, 0.02, 0.3, 1.0, 5.0], n_ids).astype(np.float32)
    part_start, part_n = 100, 300
    c = ColdDataCache(cache_size, dim, dev(hotness), cnt_threshold=3, part_start=part_start,
                      part_nnodes=part_n)
    m = O.ColdCacheServerModel(cache_size, dim, hotness, cnt_threshold=3, part_start=part_start,
                               part_nnodes=part_n)
    assert np.array_equal(c.threshold.cpu().numpy(), m.threshold.numpy())
    for step in range(30):
        if step % 3 == 0:                          # new rows arrive: evictions once the cache is full
            ids = rng.choice(n_ids, int(rng.integers(1, cache_size)), replace=False).astype(np.int64)
            embs = rng.standard_normal((ids.size, dim)).astype(np.float32)
            assert np.array_equal(c.update_cache(dev(ids), dev(embs)).cpu().numpy(),
                                  m.update_cache(ids, embs))
        ids = rng.choice(n_ids, int(rng.integers(1, 400)), replace=False).astype(np.int64)
        g = rng.standard_normal((ids.size, dim)).astype(np.float32)
        assert np.array_equal(c.accumulate_gradients_cold_remote(dev(ids), dev(g)).cpu().numpy(),
                              m.accumulate_gradients_cold_remote(ids, g))
        lids = (part_start + rng.choice(part_n, int(rng.integers(1, 100)), replace=False)).astype(np.int64)
        lg = rng.standard_normal((lids.size, dim)).astype(np.float32)
        c.accumulate_gradients_cold_local(dev(lids), dev(lg))
        m.accumulate_gradients_cold_local(lids, lg)
        _cold_state_equal(c, m)
        for got, want in ((c.staled_gradients_remote(), m.staled_gradients_remote()),
                          (c.staled_gradients_local(), m.staled_gradients_local())):
            for a, b in zip(got, want):
                assert a.cpu().numpy().dtype == b.dtype and np.array_equal(a.cpu().numpy(), b)
        _cold_state_equal(c, m)
        assert np.array_equal(c.local_grad_buff.cpu().numpy(), m.l_grad.numpy())
        assert np.array_equal(c.local_grad_cnt_buff.cpu().numpy(), m.l_cnt.numpy())
        assert np.array_equal(c.local_grad_iter_count.cpu().numpy(), m.l_iter.numpy())


def test_cold_data_cache_small_flush_capacity(lib):
    # more rows due than the output holds: the rest stays due and leaves with the next flush
    from hades_amd.cold_cache import ColdDataCache
    rng = np.random.default_rng(5)
    c = ColdDataCache(64, 4, torch.full((100,), 1000.0), cnt_threshold=1)
    ids = np.arange(40, dtype=np.int64)
    c.update_cache(dev(ids), dev(np.zeros((40, 4), np.float32)))
    g = rng.standard_normal((40, 4)).astype(np.float32)
    c.accumulate_gradients_cold_remote(dev(ids), dev(g))
    a_ids, a_g, a_c, a_n = c.staled_gradients_remote_padded(cap=25)
    b_ids, b_g, b_c, b_n = c.staled_gradients_remote_padded(cap=25)
    assert int(a_n) == 25 and int(b_n) == 15
    got = np.concatenate([a_ids[:25].cpu().numpy(), b_ids[:15].cpu().numpy()])
    rows = np.concatenate([a_g[:25].cpu().numpy(), b_g[:15].cpu().numpy()])
    order = np.argsort(got)
    assert np.array_equal(got[order], ids) and np.array_equal(rows[order], g)
    assert c.index.get_valid_entries_num() == 0 and int(c.grad_cnt_cache_buff.sum()) == 0


# ---- lookup / split -----------------------------------------------------------------------
@pytest.mark.parametrize("n,h", [(0, 10), (1, 1), (1000, 0), (4097, 511), (200_000, 48_000)])
def test_lookup_sorted(lib, n, h):
    _, ops = lib
    rng = np.random.default_rng(5 + n)
    n_rows = max(4 * h, 100)
    hot = np.sort(rng.choice(n_rows, h, replace=False)).astype(np.int64)
    q = rng.integers(-3, n_rows + 3, n).astype(np.int64)
    if n > 4 and h > 0:
        q[:4] = [hot[0], hot[-1], hot[0] - 1, hot[-1] + 1]
    loc = ops.lookup(dev(q), dev(hot))
    assert np.array_equal(loc.cpu().numpy(), O.lookup_sorted(q, hot))
    # the bucket index changes the search, never the answer
    loc = ops.lookup(dev(q), ops.HotSet(dev(hot)))
    assert np.array_equal(loc.cpu().numpy(), O.lookup_sorted(q, hot))


@pytest.mark.parametrize("kind", ["clustered", "huge_ids", "negative", "single", "dense", "zero"])
def test_lookup_bucket_index_on_awkward_id_sets(lib, kind):
    _, ops = lib
    rng = np.random.default_rng(55)
    if kind == "clustered":      # all hot ids in two narrow clusters of a wide id space
        hot = np.unique(np.concatenate([rng.integers(10**9, 10**9 + 5000, 3000),
                                        rng.integers(7, 300, 200)])).astype(np.int64)
    elif kind == "huge_ids":     # ids that need 62 bits
        hot = np.unique(rng.integers(2**61, 2**62, 4000)).astype(np.int64)
    elif kind == "negative":     # not a node-id set: the index marks itself unusable, search still right
        hot = np.unique(rng.integers(-5000, 5000, 3000)).astype(np.int64)
    elif kind == "single":
        hot = np.array([12345], np.int64)
    elif kind == "zero":
        hot = np.array([0], np.int64)
    else:                        # every id of a range
        hot = np.arange(1000, 6000, dtype=np.int64)
    extra = np.array([0, 1, -1, hot[0] - 1, hot[-1] + 1, 2**62 + 5, 2**63 - 1, -(2**63)], np.int64)
    q = np.concatenate([rng.choice(hot, 3000), rng.choice(hot, 3000) + rng.integers(-2, 3, 3000), extra])
    loc = ops.lookup(dev(q), ops.HotSet(dev(hot)))
    assert np.array_equal(loc.cpu().numpy(), O.lookup_sorted(q, hot))


@pytest.mark.parametrize("n", [0, 1, 7, 2048, 2049, 100_003])
def test_split_compact(lib, n):
    _, ops = lib
    rng = np.random.default_rng(6 + n)
    loc = np.where(rng.random(n) < 0.9, rng.integers(0, 1000, n), -1).astype(np.int64)
    hot_mask, hot_pos, cold_pos = ops.split(dev(loc))
    w_mask, w_hot, w_cold = O.split_compact(loc)
    assert hot_mask.dtype == torch.bool
    assert np.array_equal(hot_mask.cpu().numpy(), w_mask)
    assert np.array_equal(hot_pos.cpu().numpy(), w_hot)
    assert np.array_equal(cold_pos.cpu().numpy(), w_cold)


@pytest.mark.parametrize("idt", [torch.int64, torch.int32, torch.int16])
@pytest.mark.parametrize("pinned_table", [False, True])
def test_cuda_split_and_split3(lib, idt, pinned_table):
    E, ops = lib
    rng = np.random.default_rng(7)
    n_nodes = 30_000
    table = rng.integers(0, 4, n_nodes).astype(np.int8)       # value 3 belongs to no class
    ids = rng.integers(0, n_nodes, 50_001).astype(np.int64)
    t_ids = torch.from_numpy(ids).to(idt).cuda()
    if pinned_table:                                          # test/test_pin.py:24-29
        t_table = torch.empty(n_nodes, dtype=torch.int8, pin_memory=True)
        t_table.copy_(torch.from_numpy(table))
    else:
        t_table = dev(table)
    want = O.split_masks(ids, table)
    got = E.cudaSplit(t_ids, t_table)
    assert len(got) == 3 and all(g.dtype == torch.bool for g in got)
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy(), w)
    masks, pos, counts = ops.split3_padded(t_ids, t_table)
    counts = counts.tolist()
    w_masks, w_pos = O.split3_compact(ids, table)
    for k in range(3):
        assert np.array_equal(masks[k].cpu().numpy(), w_masks[k])
        assert counts[k] == w_pos[k].size
        assert np.array_equal(pos[k][:counts[k]].cpu().numpy(), w_pos[k])


# ---- cached_fetch / cached_set by the sorted hot set -----------------------------------------
@pytest.mark.parametrize("dim", [1, 64, 128, 100])
@pytest.mark.parametrize("host_cold", [False, True])
def test_cached_fetch_and_set_sorted(lib, dim, host_cold):
    _, ops = lib
    rng = np.random.default_rng(8 + dim)
    n_rows, h, n = 20_000, 3000, 7001
    shape = (n_rows,) if dim == 1 else (n_rows, dim)
    cold = rng.standard_normal(shape).astype(np.float32)
    hot_ids = np.sort(rng.choice(n_rows, h, replace=False)).astype(np.int64)
    hot = (cold[hot_ids] + 1.0).astype(np.float32)      # distinguishable from the cold copy
    q = zipfish(rng, n, n_rows)
    if host_cold:
        t_cold = torch.empty(shape, dtype=torch.float32, pin_memory=True)
        t_cold.copy_(torch.from_numpy(cold))
    else:
        t_cold = dev(cold)
    t_hot, t_q, t_ids = dev(hot), dev(q), dev(hot_ids)
    if dim != 64:
        t_ids = ops.HotSet(t_ids)       # with the bucket index; dim 64 keeps the plain binary search
    out, loc = ops.cached_fetch(t_cold, t_hot, t_q, t_ids, return_loc=True)
    assert np.array_equal(out.cpu().numpy(), O.cached_fetch(cold, hot, q, hot_ids))
    assert np.array_equal(loc.cpu().numpy(), O.lookup_sorted(q, hot_ids))
    out2 = ops.cached_fetch_loc(t_cold, t_hot, t_q, loc)
    assert torch.equal(out, out2)
    # set on duplicate-free ids
    u = np.unique(q)
    rows = rng.standard_normal((u.size,) + shape[1:]).astype(np.float32)
    w_cold, w_hot = cold.copy(), hot.copy()
    O.cached_set(rows, w_cold, w_hot, u, hot_ids)
    ops.cached_set(dev(rows), t_cold, t_hot, dev(u), t_ids)
    torch.cuda.synchronize()
    assert np.array_equal(t_cold.cpu().numpy(), w_cold)
    assert np.array_equal(t_hot.cpu().numpy(), w_hot)


# ---- combine ------------------------------------------------------------------------------
def combine_tol_ok(got, want64, scale=None):
    """tolerance mode, per row: |got - exact| <= 1e-5 * max|exact row| for every element of every
    row (exact = float64 sums).  `scale` is accepted for old call sites and ignored."""
    err = np.abs(got.astype(np.float64) - want64).max(axis=1)
    return bool(np.all(err <= 1e-5 * np.abs(want64).max(axis=1)))


CASES = [  # (n, dim, id space, kind)
    (0, 8, 100, "zipf"), (1, 8, 100, "zipf"), (2, 4, 2, "zipf"), (31, 1, 10, "zipf"),
    (32, 7, 10, "zipf"), (33, 128, 50, "zipf"), (1000, 64, 1, "same"), (4096, 128, 10**9, "distinct"),
    (5000, 100, 300, "zipf"), (20_000, 128, 2_400_000, "zipf"), (70_001, 260, 5000, "zipf"),
    (65_536, 64, 1_000_000, "zipf"),
    (3000, 7, 3, "zipf"), (2500, 1, 2, "zipf"), (40_000, 128, 40, "zipf"),   # very long runs
    # sizes either side of the sort's tile (1024), group of tiles (4096), the segmented sum's block
    # span (256) and the point where the group counts get their own scan (64 groups = 262 144 ids)
    (255, 8, 90, "zipf"), (256, 8, 90, "zipf"), (257, 8, 90, "zipf"),
    (1023, 4, 700, "zipf"), (1024, 4, 700, "zipf"), (1025, 4, 700, "zipf"),
    (4095, 4, 100_000, "zipf"), (4097, 4, 100_000, "zipf"),
    (262_144, 4, 3_000_000, "zipf"), (262_145, 4, 3_000_000, "zipf"), (530_000, 8, 50_000_000, "zipf"),
]


@pytest.fixture(params=["one_sweep", "three_kernels"])
def sort_form(request, lib):
    """runs a test once with each form of the sort under the combine; restores the default"""
    _, ops = lib
    before = ops.sort_config(one_sweep=request.param == "one_sweep")
    yield request.param
    ops.sort_config(one_sweep=before)


@pytest.mark.parametrize("n,dim,space,kind", CASES)
@pytest.mark.parametrize("bounded", [True, False])
def test_combine(lib, sort_form, n, dim, space, kind, bounded):
    _, ops = lib
    rng = np.random.default_rng(9 + n + dim)
    if kind == "same":
        idx = np.full(n, 0, np.int64)
    elif kind == "distinct":
        idx = rng.choice(space, n, replace=False).astype(np.int64)
    else:
        idx = zipfish(rng, n, space)
    if not bounded and n > 3:
        idx = idx.copy()
        idx[:3] = [-5, 2**40 + 7, -(2**50)]        # negative and wide ids: full 64-bit signed sort
    grad = (rng.standard_normal((n, dim)) * 1e-3).astype(np.float32)
    bound = space if bounded else 0
    wu, ws, wc = O.combine_sequential(idx, grad)
    if 0 < n <= 20_000:
        tu, ts, tc = O.only_unique_grads(torch.from_numpy(idx), torch.from_numpy(grad))
        assert np.array_equal(ts.numpy(), ws)       # the reference's own torch calls agree
    _, w64, _ = O.combine_float64(idx, grad)

    t_idx, t_grad = dev(idx), dev(grad)
    # deterministic-order mode: bit-equal to CPU index_add_
    uids, sums, cnts, nu, inv = ops.combine_padded(t_idx, t_grad, bound, ops.COMBINE_EXACT,
                                                   return_inverse=True)
    U = int(nu.item())
    assert U == wu.size
    assert np.array_equal(uids[:U].cpu().numpy(), wu)
    assert np.array_equal(cnts[:U].cpu().numpy(), wc)
    assert np.array_equal(sums[:U].cpu().numpy(), ws)
    if n:
        assert np.array_equal(wu[inv.cpu().numpy()], idx)
    # fast mode: ids/counts exact, sums within 1e-5 of the float64 sums, and reproducible
    uids, sums, cnts = ops.combine(t_idx, t_grad, bound, ops.COMBINE_FAST)
    assert np.array_equal(uids.cpu().numpy(), wu) and np.array_equal(cnts.cpu().numpy(), wc)
    if n:
        got = sums.cpu().numpy()
        assert combine_tol_ok(got, w64, np.abs(w64).max())
        _, sums2, _ = ops.combine(t_idx, t_grad, bound, ops.COMBINE_FAST)
        assert torch.equal(sums, sums2)
        # runs that fit inside one chunk are summed left to right: bit-equal to the exact mode
        short = wc <= 1
        assert np.array_equal(got[short], ws[short])


@pytest.mark.parametrize("dim", [4, 20, 64, 128, 7])
def test_exact_combine_long_runs_with_and_without_the_staging_area(lib, dim):
    """Deterministic-order sums of ids that occur 64 times or more: run lengths around the 64-row
    threshold and around the 1 024-row batches of the staged chain (one and two batches, one row
    more and less), a run of 40 000 rows, short runs between them, rows in shuffled batch order.
    With the full workspace the rows of the long runs are staged in column slices and summed by
    one chain per slice; with a workspace of hades_combine_workspace_bytes_min the block of a run
    fetches its rows itself.  Both equal the oracle's left-to-right sums bit for bit (dim 7: rows
    that cannot be read 16 bytes at a time take the second way whatever the workspace)."""
    from hades_amd import _lib
    _, ops = lib
    rng = np.random.default_rng(dim)
    lens = [63, 64, 65, 1, 1023, 1024, 1025, 7, 2047, 2048, 2049, 3, 3000, 40_000, 2, 100, 5000]
    idx = np.repeat(np.arange(len(lens), dtype=np.int64) * 11 + 5, lens)
    rng.shuffle(idx)
    n = idx.size
    grad = (rng.standard_normal((n, dim)) * 1e-3).astype(np.float32)
    wu, ws, wc = O.combine_sequential(idx, grad)
    t_idx, t_grad = dev(idx), dev(grad)
    full = _lib.query("hades_combine_workspace_bytes", n, dim)
    least = _lib.query("hades_combine_workspace_bytes_min", n, dim)
    assert full - least >= n * dim * 4
    st = torch.cuda.current_stream().cuda_stream
    for nbytes in (full, least):
        wsb = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        uids = torch.empty(n, dtype=torch.int64, device="cuda")
        sums = torch.full((n, dim), float("nan"), device="cuda")
        cnts = torch.empty(n, dtype=torch.int64, device="cuda")
        nu = torch.empty(1, dtype=torch.int64, device="cuda")
        for _ in range(2):      # the second call finds the list of long runs of the first one
            _lib.call("hades_combine", t_idx.data_ptr(), t_grad.data_ptr(), n, dim, 1000, ops.COMBINE_EXACT,
                      uids.data_ptr(), sums.data_ptr(), cnts.data_ptr(), nu.data_ptr(), None,
                      wsb.data_ptr(), nbytes, st)
        torch.cuda.synchronize()
        U = int(nu.item())
        assert U == wu.size and np.array_equal(uids[:U].cpu().numpy(), wu)
        assert np.array_equal(cnts[:U].cpu().numpy(), wc)
        assert np.array_equal(sums[:U].cpu().numpy(), ws)
    # one byte less than the minimum is refused
    rc = _lib.load().hades_combine(t_idx.data_ptr(), t_grad.data_ptr(), n, dim, 1000, ops.COMBINE_EXACT,
                                   uids.data_ptr(), sums.data_ptr(), cnts.data_ptr(), nu.data_ptr(), None,
                                   wsb.data_ptr(), least - 1, st)
    assert rc != 0


@pytest.mark.parametrize("n,space,bounded", [(5000, 300, True), (70_001, 5000, True), (262_145, 3_000_000, True),
                                             (150_000, 40, True), (100_000, 2_400_000, False)])
def test_one_sweep_sort_when_its_waits_run_out(lib, n, space, bounded):
    """The one-sweep sort with a spin limit of 0: every tile that finds a predecessor not ready
    gives up at once and counts the keys before it from the input itself.  The result (distinct
    ids, counts, inverse, deterministic-order sums) is that of the oracle all the same; the
    workspace's counter says how many tiles went that way; every kernel returned (the stream
    synchronises).  With the default limit the same call reports no such tile."""
    _, ops = lib
    rng = np.random.default_rng(n)
    idx = zipfish(rng, n, space)
    if not bounded:
        idx = idx.copy()
        idx[:3] = [-5, 2**40 + 7, -(2**50)]
    grad = (rng.standard_normal((n, 4)) * 1e-3).astype(np.float32)
    wu, ws, wc = O.combine_sequential(idx, grad)
    t_idx, t_grad = dev(idx), dev(grad)
    ws_buf = ops.Workspace("cuda")
    before = ops.sort_config(one_sweep=True, spin_limit=0)
    try:
        expiries = []
        for _ in range(3):
            uids, sums, cnts, nu, inv = ops.combine_padded(t_idx, t_grad, space if bounded else 0,
                                                           ops.COMBINE_EXACT, return_inverse=True,
                                                           workspace=ws_buf)
            torch.cuda.synchronize()
            expiries.append(ops.sort_wait_expiries(ws_buf))
            U = int(nu.item())
            assert U == wu.size and np.array_equal(uids[:U].cpu().numpy(), wu)
            assert np.array_equal(cnts[:U].cpu().numpy(), wc) and np.array_equal(sums[:U].cpu().numpy(), ws)
            assert np.array_equal(wu[inv.cpu().numpy()], idx)
        # with more than a handful of tiles in flight at once some tile always finds a
        # predecessor that has not published yet
        assert n < 50_000 or max(expiries) > 0
    finally:
        ops.sort_config(one_sweep=before, spin_limit=50000)
    ops.sort_config(one_sweep=True)
    try:
        uids, sums, cnts, nu = ops.combine_padded(t_idx, t_grad, space if bounded else 0, ops.COMBINE_EXACT,
                                                  workspace=ws_buf)
        torch.cuda.synchronize()
        assert ops.sort_wait_expiries(ws_buf) == 0
        assert np.array_equal(uids[:int(nu.item())].cpu().numpy(), wu)
    finally:
        ops.sort_config(one_sweep=before)


def test_rows_and_update_generated_shapes(lib):
    """Generated shapes (hypothesis) for the row kernels: any row width (vector and scalar paths,
    rows that are not a multiple of 16 bytes), any batch size, any hot fraction; fetch, set and
    the Adagrad update against the oracle, bit for bit."""
    from hypothesis import HealthCheck, given, settings, strategies as st
    _, ops = lib

    @settings(max_examples=40, deadline=None, suppress_health_check=list(HealthCheck))
    @given(st.integers(1, 300), st.integers(0, 400), st.integers(0, 60), st.integers(0, 10 ** 6))
    def run(dim, n, n_hot, seed):
        rng = np.random.default_rng(seed)
        n_rows = 500
        cold = rng.standard_normal((n_rows, dim)).astype(np.float32)
        hot_ids = np.sort(rng.choice(n_rows, n_hot, replace=False)).astype(np.int64)
        hot = rng.standard_normal((n_hot, dim)).astype(np.float32)
        q = rng.integers(0, n_rows, n).astype(np.int64)
        t_cold, t_hot, t_ids = dev(cold), dev(hot), dev(hot_ids)
        got = ops.cached_fetch(t_cold, t_hot, dev(q), t_ids)
        assert np.array_equal(got.cpu().numpy(), O.cached_fetch(cold, hot, q, hot_ids))
        u = np.unique(q)
        rows = rng.standard_normal((u.size, dim)).astype(np.float32)
        ops.cached_set(dev(rows), t_cold, t_hot, dev(u), t_ids)
        O.cached_set(rows, cold, hot, u, hot_ids)
        assert np.array_equal(t_cold.cpu().numpy(), cold) and np.array_equal(t_hot.cpu().numpy(), hot)
        cs, hs = np.abs(cold) * 0.1, np.abs(hot) * 0.1
        t_cs, t_hs = dev(cs), dev(hs)
        g = (rng.standard_normal((u.size, dim)) * 1e-2).astype(np.float32)
        ops.adagrad_update_(dev(u), dev(g), t_hot, t_hs, t_cold, t_cs, t_ids, 0.01, 1e-10)
        O.sparse_adagrad_step(cold, cs, hot, hs, hot_ids, u, g, 0.01, 1e-10)
        for a, b in ((t_cold, cold), (t_cs, cs), (t_hot, hot), (t_hs, hs)):
            assert np.array_equal(a.cpu().numpy(), b)

    run()


def test_combine_generated_batches(lib):
    """Generated small batches (hypothesis): any ids - negative, wide, heavily repeated -, any
    row width, with and without an id bound."""
    from hypothesis import HealthCheck, given, settings, strategies as st
    _, ops = lib
    wide = st.one_of(st.integers(0, 12), st.integers(0, 12), st.integers(-(2 ** 62), 2 ** 62))

    @settings(max_examples=50, deadline=None, suppress_health_check=list(HealthCheck))
    @given(st.lists(wide, min_size=0, max_size=300), st.integers(1, 9), st.booleans())
    def run(ids, dim, bounded):
        idx = np.array(ids, dtype=np.int64)
        if bounded:
            idx = np.abs(idx) % 1000
        rng = np.random.default_rng(idx.size * 31 + dim)
        grad = rng.standard_normal((idx.size, dim)).astype(np.float32)
        wu, ws, wc = O.combine_sequential(idx, grad)
        _, w64, _ = O.combine_float64(idx, grad)
        bound = 1000 if bounded else 0
        uids, sums, cnts = ops.combine(dev(idx), dev(grad), bound, ops.COMBINE_EXACT)
        assert np.array_equal(uids.cpu().numpy(), wu) and np.array_equal(cnts.cpu().numpy(), wc)
        assert np.array_equal(sums.cpu().numpy(), ws)
        uids, sums, cnts = ops.combine(dev(idx), dev(grad), bound, ops.COMBINE_FAST)
        assert np.array_equal(uids.cpu().numpy(), wu) and np.array_equal(cnts.cpu().numpy(), wc)
        if idx.size:
            assert combine_tol_ok(sums.cpu().numpy(), w64, max(np.abs(w64).max(), 1e-30))

    run()


def test_unique_grads_dropin(lib):
    from hades_amd import sparse_optim as S
    rng = np.random.default_rng(10)
    idx = zipfish(rng, 3000, 200)
    grad = rng.standard_normal((3000, 16)).astype(np.float32)
    cnt = rng.integers(1, 5, 3000).astype(np.int64)
    u, m = S.unique_grads(dev(idx), dev(grad), mode=S.ops.COMBINE_EXACT)
    wu, wm = O.unique_grads(idx, grad)
    assert np.array_equal(u.cpu().numpy(), wu.numpy())
    assert np.allclose(m.cpu().numpy(), wm.numpy(), rtol=1e-6, atol=0)
    u, m = S.unique_grads(dev(idx), dev(grad), dev(cnt), mode=S.ops.COMBINE_EXACT)
    wu, wm = O.unique_grads(idx, grad, cnt)
    assert np.array_equal(u.cpu().numpy(), wu.numpy())
    assert np.allclose(m.cpu().numpy(), wm.numpy(), rtol=1e-6, atol=0)
    u, s, c = S.only_unique_grads(dev(idx), dev(grad), mode=S.ops.COMBINE_EXACT)
    wu, ws, wc = O.only_unique_grads(idx, grad)
    assert torch.equal(s.cpu(), ws) and torch.equal(c.cpu(), wc) and torch.equal(u.cpu(), wu)


# ---- row optimizers -------------------------------------------------------------------------
@pytest.mark.parametrize("dim", [64, 128, 7])
@pytest.mark.parametrize("host_cold", [False, True])
def test_adagrad_update(lib, dim, host_cold):
    _, ops = lib
    rng = np.random.default_rng(11 + dim)
    n_rows, h = 30_000, 4000
    cw = (rng.standard_normal((n_rows, dim)) * 0.01).astype(np.float32)
    cs = np.zeros((n_rows, dim), np.float32)
    hot_ids = np.sort(rng.choice(n_rows, h, replace=False)).astype(np.int64)
    hw, hs = cw[hot_ids].copy(), cs[hot_ids].copy()

    def place(a):
        if host_cold:
            t = torch.empty(a.shape, dtype=torch.float32, pin_memory=True)
            t.copy_(torch.from_numpy(a))
            return t
        return dev(a)
    t_cw, t_cs, t_hw, t_hs, t_ids = place(cw), place(cs), dev(hw), dev(hs), dev(hot_ids)
    for step in range(3):
        u = np.unique(zipfish(rng, 9000, n_rows))
        g = (rng.standard_normal((u.size, dim)) * 1e-3).astype(np.float32)
        O.sparse_adagrad_step(cw, cs, hw, hs, hot_ids, u, g, 0.01, 1e-10)
        # pad the device batch and pass the live count from device memory
        pad = 100
        t_u = dev(np.concatenate([u, np.zeros(pad, np.int64)]))
        t_g = dev(np.concatenate([g, np.ones((pad, dim), np.float32)]))
        nu = torch.tensor([u.size], dtype=torch.int64, device="cuda")
        ops.adagrad_update_(t_u, t_g, t_hw, t_hs, t_cw, t_cs, t_ids, 0.01, 1e-10, num_unique=nu)
        torch.cuda.synchronize()
        for got, want in ((t_cw, cw), (t_cs, cs), (t_hw, hw), (t_hs, hs)):
            assert np.array_equal(got.cpu().numpy(), want)      # one rounding per operation: bit-exact


def test_adagrad_vs_torch_optim(lib):
    """The same update against torch.optim.Adagrad on a dense parameter: <= 1e-5 relative."""
    _, ops = lib
    rng = np.random.default_rng(12)
    n_rows, dim = 2000, 32
    w0 = (rng.standard_normal((n_rows, dim)) * 0.01).astype(np.float32)
    p = torch.nn.Parameter(torch.from_numpy(w0.copy()))
    opt = torch.optim.Adagrad([p], lr=0.01, eps=1e-10)
    t_w, t_s = dev(w0), torch.zeros((n_rows, dim), device="cuda")
    for _ in range(3):
        u = np.unique(rng.integers(0, n_rows, 700))
        g = (rng.standard_normal((u.size, dim)) * 1e-3).astype(np.float32)
        dense = np.zeros_like(w0)
        dense[u] = g
        p.grad = torch.from_numpy(dense)
        opt.step()
        ops.adagrad_update_(dev(u), dev(g), None, None, t_w, t_s, None, 0.01, 1e-10)
    assert np.allclose(t_w.cpu().numpy(), p.detach().numpy(), rtol=1e-5, atol=1e-9)


def test_adam_update(lib):
    _, ops = lib
    rng = np.random.default_rng(13)
    n_rows, h, dim = 8000, 1000, 64
    w = (rng.standard_normal((n_rows, dim)) * 0.01).astype(np.float32)
    st = np.zeros(n_rows, np.float32); m = np.zeros_like(w); v = np.zeros_like(w)
    hot_ids = np.sort(rng.choice(n_rows, h, replace=False)).astype(np.int64)
    t_cold = tuple(dev(x) for x in (w, st, m, v))
    t_hot = tuple(dev(x[hot_ids]) for x in (w, st, m, v))
    t_ids = dev(hot_ids)
    for _ in range(3):
        u = np.unique(zipfish(rng, 3000, n_rows))
        g = (rng.standard_normal((u.size, dim)) * 1e-2).astype(np.float32)
        w[u], st[u], m[u], v[u] = O.adam_rows(w[u], st[u], m[u], v[u], g, 0.01, 0.9, 0.999, 1e-8)
        ops.adam_update_(dev(u), dev(g), t_hot, t_cold, t_ids, 0.01, 0.9, 0.999, 1e-8)
    torch.cuda.synchronize()
    for k, want in enumerate((w, st, m, v)):
        got = t_cold[k].cpu().numpy()
        got[hot_ids] = t_hot[k].cpu().numpy()
        if k == 0:
            # powf differs by an ulp between host and device and 1 - 0.999^t amplifies it:
            # compare to 1e-4 of one update (lr = 0.01)
            assert np.abs(got - want).max() <= 1e-4 * 0.01
        elif k == 1:
            assert np.array_equal(got, want)
        else:
            assert np.allclose(got, want, rtol=1e-6, atol=1e-12)


@pytest.mark.parametrize("variant", ["duplicates", "duplicates_cnt", "unique_cnt"])
def test_sparse_adam_like_reference(lib, variant):
    """SparseAdam.update_like_reference against the reference's update restated by the oracle:
    unique_grads (mean over duplicates, the count quirk with cnt) or the is_unique branch, then
    adam_rows on the gathered rows (python/EmbCache/sparse_optim.py:590-685)."""
    from hades_amd.sparse_optim import SparseAdam
    rng = np.random.default_rng(17)
    n_rows, h, dim = 6000, 800, 32
    w = (rng.standard_normal((n_rows, dim)) * 0.01).astype(np.float32)
    st = np.zeros(n_rows, np.float32); m = np.zeros_like(w); v = np.zeros_like(w)
    hot_ids = np.sort(rng.choice(n_rows, h, replace=False)).astype(np.int64)
    opt = SparseAdam(dev(w), dev(hot_ids), lr=0.01, betas=(0.9, 0.999), eps=1e-8)
    for _ in range(3):
        idx = zipfish(rng, 2500, n_rows)
        if variant == "unique_cnt":
            idx = np.unique(idx)
        g = (rng.standard_normal((idx.size, dim)) * 1e-2).astype(np.float32)
        cnt = None if variant == "duplicates" else rng.integers(1, 6, idx.size).astype(np.int64)
        if variant == "unique_cnt":
            u, vals = idx, g / cnt[:, None].astype(np.float32)                  # :607-611
        else:
            tu, tv = O.unique_grads(idx, g, cnt)                                # :613
            u, vals = tu.numpy(), tv.numpy()
        w[u], st[u], m[u], v[u] = O.adam_rows(w[u], st[u], m[u], v[u], vals, 0.01, 0.9, 0.999, 1e-8)
        got_u = opt.update_like_reference(dev(idx), dev(g), None if cnt is None else dev(cnt),
                                          is_unique=(variant == "unique_cnt"), mode=ops_exact(lib))
        assert np.array_equal(got_u.cpu().numpy(), u)
    torch.cuda.synchronize()
    for k, (cold, hot, want) in enumerate(((opt.cold_w, opt.hot_w, w), (opt.cold_step, opt.hot_step, st),
                                           (opt.cold_m, opt.hot_m, m), (opt.cold_v, opt.hot_v, v))):
        got = cold.cpu().numpy().copy()
        got[hot_ids] = hot.cpu().numpy()
        if k == 0:
            assert np.abs(got - want).max() <= 1e-4 * 0.01      # as in test_adam_update
        elif k == 1:
            assert np.array_equal(got, want)
        else:
            assert np.allclose(got, want, rtol=1e-6, atol=1e-12)


def ops_exact(lib):
    return lib[1].COMBINE_EXACT


# ---- cold-gradient accumulator ------------------------------------------------------------------
@pytest.mark.parametrize("dim", [128, 5])
def test_hash_accumulator(lib, dim):
    _, ops = lib
    rng = np.random.default_rng(14 + dim)
    acc = ops.ColdGradAccumulator(num_slots=4096, dim=dim, id_bound=10**6)
    model = O.ColdGradAccumulatorModel(dim)
    for rounds in range(2):
        for step in range(4):
            ids = np.minimum(rng.pareto(0.5, 900).astype(np.int64), 10**6 - 1)
            g = (rng.standard_normal((900, dim)) * 1e-3).astype(np.float32)
            u, s, c = O.combine_sequential(ids, g)
            model.accumulate(u, s, c)
            uids, sums, cnts, nu = ops.combine_padded(dev(ids), dev(g), 10**6, ops.COMBINE_EXACT)
            acc.accumulate(uids, sums, cnts, num_rows=nu)
        wi, ws, wc = model.flush()
        gi, gs, gc = acc.flush(cap=4096)
        assert np.array_equal(gi.cpu().numpy(), wi)
        assert np.array_equal(gc.cpu().numpy(), wc)
        assert np.array_equal(gs.cpu().numpy(), ws)   # one add per slot per step, in step order
    gi, _, _ = acc.flush(cap=4096)
    assert gi.numel() == 0
    assert bool((acc.keys == -1).all()) and float(acc.accum.abs().sum()) == 0.0


def test_hash_accumulator_overflow_is_reported(lib):
    _, ops = lib
    acc = ops.ColdGradAccumulator(num_slots=64, dim=4)
    ids = torch.arange(100, dtype=torch.int64, device="cuda")
    acc.accumulate(ids, torch.ones((100, 4), device="cuda"))
    with pytest.raises(RuntimeError):
        acc.flush()


# ---- the whole step at benchmark size: properties that do not need the oracle --------------------
def test_full_size_step_properties(lib):
    _, ops = lib
    from hades_amd import synth
    from hades_amd.sparse_optim import SparseAdagrad
    cfg = synth.CONFIGS["cfg2"]
    N, D, H, n = cfg["num_rows"], cfg["dim"], cfg["num_hot"], cfg["batch"]
    table = torch.empty((N, D), device="cuda")
    synth.fill_normal_(table, 0.01, 1)
    hot_ids = synth.hot_ids(N, H, "cuda")
    opt = SparseAdagrad(table, hot_ids, lr=0.01, eps=1e-10)
    sampler = synth.ZipfSampler(N, cfg["zipf_s"], "cuda")
    q = synth.make_ids(sampler, N, n, 7)
    grad = synth.make_grads(n, D, 8, "cuda")
    # fetch agrees with plain indexing of the merged table (hot copy == cold copy before any update)
    rows = opt.fetch(q)
    assert torch.equal(rows, table[q])
    loc = ops.lookup(q, hot_ids)
    hit = loc >= 0
    assert torch.equal(hot_ids[loc[hit]], q[hit])
    assert not torch.isin(q[~hit], hot_ids).any()
    hot_mask, hot_pos, cold_pos = ops.split(loc)
    assert torch.equal(hot_mask, hit)
    assert torch.equal(hot_pos, torch.nonzero(hit).flatten())
    assert torch.equal(cold_pos, torch.nonzero(~hit).flatten())
    # combine: torch's own unique/index_add_ on the device as an independent check
    uids, sums, cnts, nu = opt.step(q, grad)
    U = int(nu.item())
    tu, tinv, tc = torch.unique(q, return_inverse=True, return_counts=True)
    assert U == tu.numel() and torch.equal(uids[:U], tu) and torch.equal(cnts[:U], tc)
    ref = torch.zeros((U, D), dtype=torch.float64, device="cuda").index_add_(0, tinv, grad.double())
    assert (sums[:U].double() - ref).abs().max().item() <= 1e-5 * ref.abs().max().item()
    assert int(cnts[:U].sum()) == n
    # update touched exactly the rows of uids, hot rows in the hot copy only
    uloc = ops.lookup(uids[:U], hot_ids)
    cold_u = uids[:U][uloc < 0]
    changed = (opt.cold_s.abs().sum(1) > 0).nonzero().flatten()
    assert torch.equal(changed, cold_u)
    hot_changed = (opt.hot_s.abs().sum(1) > 0).nonzero().flatten()
    assert torch.equal(hot_changed, torch.sort(uloc[uloc >= 0]).values)
    g = sums[:U][uloc < 0]
    assert torch.equal(opt.cold_s[cold_u], g * g)      # first step from a zero accumulator


def test_full_size_local_aggregation_and_accumulator_round_trip(lib):
    """cfg5's shape (four trainers' 256 K-id batches over a 244 M-row id space, 64 columns) and
    cfg4's (512 K cold ids per step into a 4 M-slot accumulator), through properties that need no
    oracle: agreement with torch's own device unique / index_add_, combine(concat(batches)) ==
    combine(concat(combine(batch_t))), and flush(accumulate(batches)) == combine(concat(batches))."""
    _, ops = lib
    from hades_amd import synth
    c5 = synth.CONFIGS["cfg5"]
    N, D, T, b = c5["num_rows"], c5["dim"], c5["trainers"], c5["batch"]
    sampler = synth.ZipfSampler(N, c5["zipf_s"], "cuda")
    qs = [synth.make_ids(sampler, N, b, 40 + t) for t in range(T)]
    gs = [synth.make_grads(b, D, 50 + t, "cuda") for t in range(T)]
    del sampler
    q, g = torch.cat(qs), torch.cat(gs)
    uids, sums, cnts = ops.combine(q, g, id_bound=N)
    tu, tinv, tc = torch.unique(q, return_inverse=True, return_counts=True)
    assert torch.equal(uids, tu) and torch.equal(cnts, tc) and int(cnts.sum()) == T * b
    ref = torch.zeros((tu.numel(), D), dtype=torch.float64, device="cuda").index_add_(0, tinv, g.double())
    scale = ref.abs().max().item()
    assert (sums.double() - ref).abs().max().item() <= 1e-5 * scale
    # two-level aggregation: per-trainer combine first, then the combine of the partial results
    parts = [ops.combine(qs[t], gs[t], id_bound=N) for t in range(T)]
    u2, s2, _ = ops.combine(torch.cat([p[0] for p in parts]), torch.cat([p[1] for p in parts]), id_bound=N)
    assert torch.equal(u2, uids)
    assert (s2.double() - ref).abs().max().item() <= 1e-5 * scale
    del ref, sums, s2, parts, q, g, qs, gs

    c4 = synth.CONFIGS["cfg4"]
    N4, H4, D4, n4 = c4["num_rows"], c4["num_hot"], c4["dim"], c4["batch"]
    sampler = synth.ZipfSampler(N4 - H4, c4["zipf_s"], "cuda")
    acc = ops.ColdGradAccumulator(c4["num_slots"], D4, id_bound=N4, device="cuda")
    all_ids, all_g, all_c = [], [], []
    for step in range(c4["flush_every"]):
        ids = synth.make_ids(sampler, N4, n4, 60 + step, rank_offset=H4)
        grad = synth.make_grads(n4, D4, 70 + step, "cuda")
        u, s, c = ops.combine(ids, grad, id_bound=N4, mode=ops.COMBINE_EXACT)
        acc.accumulate(u, s, c)
        all_ids.append(u); all_g.append(s); all_c.append(c)
    f_ids, f_sums, f_cnts = acc.flush()
    cat_ids, cat_g, cat_c = torch.cat(all_ids), torch.cat(all_g), torch.cat(all_c)
    tu, tinv = torch.unique(cat_ids, return_inverse=True)
    assert torch.equal(f_ids, tu) and (f_ids >= 0).all()
    want_c = torch.zeros(tu.numel(), dtype=torch.int64, device="cuda").index_add_(0, tinv, cat_c)
    assert torch.equal(f_cnts, want_c) and int(f_cnts.sum()) == c4["flush_every"] * n4
    # one add per slot per step in step order: the same float32 chain as combining the
    # concatenated per-step results in EXACT mode
    e_ids, e_sums, _ = ops.combine(cat_ids, cat_g, id_bound=N4, mode=ops.COMBINE_EXACT)
    assert torch.equal(e_ids, f_ids) and torch.equal(e_sums, f_sums)
    assert acc.flush()[0].numel() == 0                      # the table is empty again


@pytest.mark.parametrize("pinned", [False, True])
def test_emb_cache_state_tables(lib, pinned):
    """EmbCache over the three tables of the reference's state cache (step [N], mem [N, D],
    power [N, D]; python/EmbCache/cache.py:66-131): budgeted hotness placement, getitem / setitem
    against plain indexing of a merged reference copy, hit rate, write-back."""
    from hades_amd.cache import EmbCache
    rng = np.random.default_rng(9)
    N, D = 20_000, 32
    mk = (lambda *s: torch.zeros(*s, pin_memory=True)) if pinned else (lambda *s: torch.zeros(*s, device="cuda"))
    tables = [mk(N), mk(N, D), mk(N, D)]
    for t in tables:
        t.copy_(torch.from_numpy(rng.standard_normal(tuple(t.shape)).astype(np.float32)))
    ref = [t.clone().cpu().numpy() for t in tables]
    hotness = torch.from_numpy(rng.random(N).astype(np.float32))
    item = 4 + 4 * D + 4 * D + 8
    cache = EmbCache.create_cache(tables, hotness, alloca_mem_size=3000 * item + 5, count_hit=True)
    want_hot = O.select_hot_ids(hotness, 3000)
    assert np.array_equal(cache.hot_ids.cpu().numpy(), want_hot)
    for step in range(3):
        q = rng.integers(0, N, 4000).astype(np.int64)
        got = cache[dev(q)]
        for k in range(3):
            assert np.array_equal(got[k].cpu().numpy(), ref[k][q])
        u = np.unique(rng.integers(0, N, 3000)).astype(np.int64)
        vals = [rng.standard_normal((u.size,) + r.shape[1:]).astype(np.float32) for r in ref]
        cache[dev(u)] = tuple(dev(v) for v in vals)
        for k in range(3):
            ref[k][u] = vals[k]
    hits = sum(int(np.isin(q_, want_hot).sum()) for q_ in [q])      # last batch, as a sanity bound
    assert 0.0 < cache.get_hit_rate() < 1.0 and hits > 0
    # cached rows live in the hot copy only until written back
    torch.cuda.synchronize()
    hot_changed = np.isin(u, want_hot)
    if hot_changed.any():
        k0 = u[hot_changed][0]
        assert not np.array_equal(tables[1][k0].cpu().numpy(), ref[1][k0])
    cache.write_back()
    torch.cuda.synchronize()
    for k in range(3):
        assert np.array_equal(tables[k].cpu().numpy(), ref[k])


def test_step_replayed_from_a_hip_graph_matches_eager(lib):
    """The library allocates nothing, synchronises nothing and clears memory with kernels only, so
    a whole step can be captured once and replayed.  Every replay - with fresh inputs copied into
    the captured buffers and eager work of the same library in between - must give exactly what
    the eager step gives from the same state."""
    _, ops = lib
    from hades_amd.sparse_optim import SparseAdagrad
    rng = np.random.default_rng(77)
    N, D, H, n = 50_000, 64, 5_000, 20_000
    table0 = torch.from_numpy((rng.standard_normal((N, D)) * 0.01).astype(np.float32)).cuda()
    hot_ids = torch.from_numpy(np.sort(rng.choice(N, H, replace=False)).astype(np.int64)).cuda()
    batches = [(dev(zipfish(rng, n, N)), dev((rng.standard_normal((n, D)) * 1e-3).astype(np.float32)))
               for _ in range(4)]

    def make():
        opt = SparseAdagrad(table0.clone(), hot_ids, lr=0.01, eps=1e-10)
        bufs = dict(rows=torch.empty((n, D), device="cuda"),
                    comb=(torch.empty(n, dtype=torch.int64, device="cuda"),
                          torch.empty((n, D), device="cuda"),
                          torch.empty(n, dtype=torch.int64, device="cuda"),
                          torch.empty(1, dtype=torch.int64, device="cuda")))
        return opt, bufs

    def step(opt, bufs, q, g):
        ops.cached_fetch(opt.cold_w, opt.hot_w, q, opt.hot_set, out=bufs["rows"])
        plan = ops.combine_plan(q, D, id_bound=N, workspace=opt._ws,
                                out=(bufs["comb"][0], bufs["comb"][3]))
        uids, sums, cnts, nu = ops.combine_apply(plan, g, ops.COMBINE_FAST,
                                                 out=(bufs["comb"][1], bufs["comb"][2]))
        opt.update(uids, sums, nu)

    eager, ebufs = make()
    graphed, gbufs = make()
    q_in, g_in = batches[0][0].clone(), batches[0][1].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(graphed, gbufs, q_in, g_in)           # warm-up on the capture stream: workspaces exist
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step(graphed, gbufs, q_in, g_in)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    # the warm-up changed the graphed optimizer once with batch 0: bring the eager one level
    step(eager, ebufs, *batches[0])
    for i in range(6):
        q, g = batches[i % 4]
        step(eager, ebufs, q, g)
        q_in.copy_(q); g_in.copy_(g)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(gbufs["rows"], ebufs["rows"])
        u = int(ebufs["comb"][3].item())
        assert int(gbufs["comb"][3].item()) == u
        for k in range(3):
            assert torch.equal(gbufs["comb"][k][:u], ebufs["comb"][k][:u])
        for name in ("cold_w", "cold_s", "hot_w", "hot_s"):
            assert torch.equal(getattr(graphed, name), getattr(eager, name)), (i, name)
        # eager work of the same library between replays
        ops.lookup(q, graphed.hot_set)
        ops.combine(q[:1000], g[:1000], id_bound=N)


def test_combine_plan_then_apply_and_side_stream_schedule(lib):
    """The two halves of combine give what the whole gives; a plan made on a side stream while the
    main stream fetches gives the same optimizer step as the one-stream order."""
    _, ops = lib
    from hades_amd.sparse_optim import SparseAdagrad
    rng = np.random.default_rng(77)
    n_rows, dim, n = 60_000, 64, 50_000
    idx = zipfish(rng, n, n_rows)
    grad = (rng.standard_normal((n, dim)) * 1e-3).astype(np.float32)
    t_idx, t_grad = dev(idx), dev(grad)
    for mode in (ops.COMBINE_EXACT, ops.COMBINE_FAST):
        whole = ops.combine_padded(t_idx, t_grad, n_rows, mode)
        plan = ops.combine_plan(t_idx, dim, n_rows)
        halves = ops.combine_apply(plan, t_grad, mode)
        U = int(whole[3].item())
        assert U == int(halves[3].item())
        for a, b in zip(whole[:3], halves[:3]):
            assert torch.equal(a[:U], b[:U])
    table = (rng.standard_normal((n_rows, dim)) * 0.01).astype(np.float32)
    hot_ids = np.sort(rng.choice(n_rows, 6000, replace=False)).astype(np.int64)
    a = SparseAdagrad(dev(table), torch.from_numpy(hot_ids))
    b = SparseAdagrad(dev(table), torch.from_numpy(hot_ids))
    for step in range(3):
        idx = zipfish(rng, n, n_rows)
        t_idx = dev(idx)
        t_grad = dev((rng.standard_normal((n, dim)) * 1e-3).astype(np.float32))
        a.fetch(t_idx)
        a.step(t_idx, t_grad)
        plan = b.prepare(t_idx)          # side stream
        rows = b.fetch(t_idx)            # main stream, concurrently
        b.step(t_idx, t_grad, plan=plan)
        del rows
    torch.cuda.synchronize()
    for x, y in ((a.cold_w, b.cold_w), (a.cold_s, b.cold_s), (a.hot_w, b.hot_w), (a.hot_s, b.hot_s)):
        assert torch.equal(x, y)


def test_combine_reports_an_id_outside_its_bound(lib):
    """An id outside [0, id_bound) cannot be sorted over the shortened key: the combine then says
    -1 distinct ids, the trimmed forms raise, and an update driven by that count touches nothing."""
    _, ops = lib
    from hades_amd import sparse_optim
    rng = np.random.default_rng(5)
    n, dim, bound = 30_000, 16, 1000
    idx = rng.integers(0, bound, n).astype(np.int64)
    grad = rng.standard_normal((n, dim)).astype(np.float32)
    for bad_id in (bound, -1, 2**40):
        bad = idx.copy()
        bad[n // 3] = bad_id
        out = ops.combine_padded(dev(bad), dev(grad), bound)
        assert int(out[3].item()) == -1
        with pytest.raises(RuntimeError, match="id_bound"):
            ops.combine(dev(bad), dev(grad), bound)
        with pytest.raises(RuntimeError, match="id_bound"):
            sparse_optim.unique_grads(dev(bad), dev(grad), id_bound=bound)
        w = torch.ones((bound, dim), device="cuda")
        s = torch.zeros((bound, dim), device="cuda")
        ops.adagrad_update_(out[0], out[1], None, None, w, s, None, 0.01, 1e-10, num_unique=out[3])
        assert bool((w == 1).all()) and bool((s == 0).all())
        ops.rows_div_count_(out[1], out[2], out[3])
    # the same workspace serves a good batch afterwards (nothing sticks)
    uids, sums, cnts = ops.combine(dev(idx), dev(grad), bound, ops.COMBINE_EXACT)
    wu, ws, wc = O.combine_sequential(idx, grad)
    assert np.array_equal(uids.cpu().numpy(), wu) and np.array_equal(sums.cpu().numpy(), ws)
    # without a bound the same ids are fine
    bad = idx.copy(); bad[7] = -1
    uids, _, _ = ops.combine(dev(bad), dev(grad), 0)
    assert int(uids[0]) == -1


def test_combine_plan_is_invalidated_by_a_later_plan(lib):
    _, ops = lib
    ws = ops.Workspace("cuda")
    idx = torch.arange(1000, dtype=torch.int64, device="cuda") % 10
    grad = torch.ones((1000, 4), device="cuda")
    p1 = ops.combine_plan(idx, 4, 10, workspace=ws)
    p2 = ops.combine_plan(idx, 4, 10, workspace=ws)
    with pytest.raises(RuntimeError, match="invalidated"):
        ops.combine_apply(p1, grad)
    assert int(ops.combine_apply(p2, grad)[3].item()) == 10
    p3 = ops.combine_plan(idx, 4, 10, workspace=ws)
    big = torch.arange(100_000, dtype=torch.int64, device="cuda")
    ops.combine_plan(big, 4, 0, workspace=ws)            # grows the buffer
    with pytest.raises(RuntimeError, match="invalidated"):
        ops.combine_apply(p3, grad)


def test_accumulator_rejects_negative_ids(lib):
    """-1 marks an empty slot: a negative id is dropped and reported, it never takes a slot."""
    _, ops = lib
    acc = ops.ColdGradAccumulator(num_slots=1024, dim=8, id_bound=10**6)
    ids = dev(np.array([5, -1, 77, -9], np.int64))
    grad = torch.ones((4, 8), device="cuda")
    acc.accumulate(ids, grad)
    assert int(acc.status.item()) == 8
    acc.status.zero_()
    f_ids, f_sums, f_cnts = acc.flush()
    assert f_ids.tolist() == [5, 77] and f_cnts.tolist() == [1, 1]
    assert bool((f_sums == 1).all())


# ---- the split schedule: lookup + partition, then one kernel per class -------------------
def _split_case(rng, N, D, H, n, hot_frac):
    """ids with a chosen share of hot ones; hot copies differ from the cold copies so that a row's
    source shows in its value."""
    cold = (rng.standard_normal((N, D)) * 0.01).astype(np.float32)
    hot_ids = np.sort(rng.choice(N, H, replace=False)).astype(np.int64) if H else np.zeros(0, np.int64)
    cold_ids = np.setdiff1d(np.arange(N, dtype=np.int64), hot_ids)
    is_hot = rng.random(n) < hot_frac
    if H == 0:
        is_hot[:] = False
    if cold_ids.size == 0:
        is_hot[:] = True
    q = np.where(is_hot, hot_ids[rng.integers(0, max(H, 1), n)] if H else 0,
                 cold_ids[rng.integers(0, max(cold_ids.size, 1), n)] if cold_ids.size else 0).astype(np.int64)
    return cold, hot_ids, q


@pytest.mark.parametrize("N,D,H,n,hot_frac", [
    (5000, 128, 500, 20_000, 0.9),      # the usual mix
    (5000, 64, 500, 20_000, 1.0),       # all hot: the cold class is empty
    (5000, 64, 500, 20_000, 0.0),       # all cold: the hot class is empty
    (5000, 7, 0, 3000, 0.0),            # no hot set at all, scalar row path
    (300, 100, 300, 4097, 1.0),         # every id hot
    (70_000, 128, 9000, 2049, 0.5), (70_000, 128, 9000, 2048, 0.5), (70_000, 128, 9000, 1, 0.5),
    (10, 4, 3, 0, 0.5),                 # empty batch
])
@pytest.mark.parametrize("host_cold", [False, True])
def test_split_schedule_fetch_and_update(lib, N, D, H, n, hot_frac, host_cold):
    _, ops = lib
    from hades_amd.sparse_optim import SparseAdagrad
    rng = np.random.default_rng(N + n + int(10 * hot_frac))
    cold, hot_ids, q = _split_case(rng, N, D, H, n, hot_frac)
    t_cold = torch.from_numpy(cold.copy())
    t_cold = t_cold.pin_memory() if host_cold else t_cold.cuda()
    opt = SparseAdagrad(t_cold, torch.from_numpy(hot_ids), lr=0.01, eps=1e-10)
    opt.hot_w += 1.0                                     # hot copy != cold copy from here on
    hw = opt.hot_w.cpu().numpy().copy()
    # lookup + partition
    t_q = dev(q)
    loc, hot_pos, cold_pos, counts = ops.lookup_split(t_q, opt.hot_set)
    w_loc, w_hp, w_cp = O.lookup_split(q, hot_ids)
    nh, nc = counts.tolist()
    assert (nh, nc) == (w_hp.size, w_cp.size)
    assert np.array_equal(loc.cpu().numpy(), w_loc)
    assert np.array_equal(hot_pos[:nh].cpu().numpy(), w_hp) and np.array_equal(cold_pos[:nc].cpu().numpy(), w_cp)
    # fetch, class by class on two streams == the oracle's cached_fetch == the one-kernel fetch
    want = O.cached_fetch(cold, hw, q, hot_ids)
    got = opt.fetch_split(t_q)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), want)
    if n:
        assert torch.equal(got, ops.cached_fetch(opt.cold_w, opt.hot_w, t_q, opt.hot_set))
    # update: combine (EXACT), then the class-by-class Adagrad == oracle, bit for bit
    grad = (rng.standard_normal((n, D)) * 1e-3).astype(np.float32)
    cw, cs = cold.copy(), np.zeros_like(cold)
    hs = np.zeros_like(hw)
    for _ in range(2):
        uids, sums, cnts, nu = opt.step_split(t_q, dev(grad), mode=ops.COMBINE_EXACT)
        wu, ws, _ = O.combine_sequential(q, grad)
        O.sparse_adagrad_step(cw, cs, hw, hs, hot_ids, wu, ws, 0.01, 1e-10)
    torch.cuda.synchronize()
    assert np.array_equal(opt.cold_w.cpu().numpy(), cw) and np.array_equal(opt.cold_s.cpu().numpy(), cs)
    assert np.array_equal(opt.hot_w.cpu().numpy(), hw) and np.array_equal(opt.hot_s.cpu().numpy(), hs)


def test_listed_operators_partial_counts_and_strided_tables(lib):
    """fetch_listed / set_listed / adagrad_update_listed_ with a device-side count below, at and
    above the list length, a negative count, and a host table whose weight and state rows are
    interleaved ([N, 2, D]: one burst per row over the host link)."""
    _, ops = lib
    rng = np.random.default_rng(8)
    N, D, n = 4000, 128, 3000
    both = torch.empty((N, 2, D), dtype=torch.float32).pin_memory()
    both.copy_(torch.from_numpy(rng.standard_normal((N, 2, D)).astype(np.float32)))
    both[:, 1].abs_()
    w, s = both[:, 0], both[:, 1]                       # row stride 2 * D
    ref = both.numpy().copy()
    idx = rng.permutation(N)[:n].astype(np.int64)
    pos = rng.permutation(n).astype(np.int64)
    t_idx, t_pos = dev(idx), dev(pos)
    for count in (0, 1, 777, n, n + 5, -1):
        live = max(0, min(count, n))
        t_count = torch.tensor([count], dtype=torch.int64, device="cuda")
        out = torch.full((n, D), -7.0, device="cuda")
        ops.fetch_listed(w, t_idx, t_pos, t_count, out)
        want = O.fetch_listed(ref[:, 0], idx, pos, live, np.full((n, D), -7.0, np.float32))
        assert np.array_equal(out.cpu().numpy(), want)
        g = (rng.standard_normal((n, D)) * 1e-3).astype(np.float32)
        ops.adagrad_update_listed_(t_idx, dev(g), t_pos, t_count, w, s, 0.01, 1e-10)
        rw, rs = ref[:, 0].copy(), ref[:, 1].copy()
        O.adagrad_listed(idx, g, pos, live, rw, rs, 0.01, 1e-10)
        ref[:, 0], ref[:, 1] = rw, rs
        torch.cuda.synchronize()
        assert np.array_equal(both.numpy(), ref)
        src = np.abs(rng.standard_normal((n, D))).astype(np.float32)     # a state row: >= 0
        ops.set_listed(dev(src), s, t_idx, t_pos, t_count)
        rs = ref[:, 1].copy()
        O.set_listed(src, rs, idx, pos, live)
        ref[:, 1] = rs
        torch.cuda.synchronize()
        assert np.array_equal(both.numpy(), ref)
    # the optimizer on the interleaved host table: split schedule, hot copies in HBM
    hot_ids = np.sort(rng.choice(N, 300, replace=False)).astype(np.int64)
    from hades_amd.sparse_optim import SparseAdagrad
    both[:, 1].zero_()
    ref = both.numpy().copy()
    opt = SparseAdagrad(w, torch.from_numpy(hot_ids), cold_state=s)
    q = rng.integers(0, N, 10_000).astype(np.int64)
    grad = (rng.standard_normal((q.size, D)) * 1e-3).astype(np.float32)
    rows = opt.fetch_split(dev(q))
    assert np.array_equal(rows.cpu().numpy(), ref[:, 0][q])
    opt.step_split(dev(q), dev(grad), mode=ops.COMBINE_EXACT)
    torch.cuda.synchronize()
    cw, cs = ref[:, 0].copy(), ref[:, 1].copy()
    hw, hs = cw[hot_ids].copy(), cs[hot_ids].copy()
    wu, ws, _ = O.combine_sequential(q, grad)
    O.sparse_adagrad_step(cw, cs, hw, hs, hot_ids, wu, ws, 0.01, 1e-10)
    assert np.array_equal(both[:, 0].numpy(), cw) and np.array_equal(both[:, 1].numpy(), cs)
    assert np.array_equal(opt.hot_w.cpu().numpy(), hw) and np.array_equal(opt.hot_s.cpu().numpy(), hs)


# ---- pinning and the library's own pinned allocation (src/cuda/pin_memory.cu:9-26) -------------
def test_library_pinned_allocation_through_the_c_abi(lib):
    """hades_host_alloc -> fill from the host -> hades_fetch2 / hades_set / hades_cached_fetch /
    hades_adagrad_update on that memory -> oracle -> hades_host_free, all through the C ABI with
    raw pointers."""
    import ctypes
    from hades_amd import _lib
    L = _lib.load()
    rng = np.random.default_rng(404)
    N, D, n = 20_000, 96, 5_000
    nbytes = N * D * 4
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for flags in (0, _lib.HOST_NONCOHERENT):
        raw = ctypes.c_void_p()
        _lib.call("hades_host_alloc_flags", ctypes.byref(raw), nbytes, flags)
        assert raw.value
        host = np.ctypeslib.as_array((ctypes.c_float * (N * D)).from_address(raw.value)).reshape(N, D)
        host[:] = rng.standard_normal((N, D)).astype(np.float32)          # filled by the CPU
        want_tab = host.copy()
        idx = rng.permutation(N)[:n].astype(np.int64)
        t_idx = dev(idx)
        # gather out of the host table
        out = torch.empty((n, D), device="cuda")
        _lib.call("hades_fetch2", raw, ctypes.c_void_p(t_idx.data_ptr()), ctypes.c_void_p(out.data_ptr()),
                  n, D, _lib.F32, _lib.I64, st)
        assert np.array_equal(out.cpu().numpy(), O.fetch2(want_tab, idx))
        # scatter into it
        src = rng.standard_normal((n, D)).astype(np.float32)
        t_src = dev(src)
        _lib.call("hades_set", ctypes.c_void_p(t_src.data_ptr()), raw, ctypes.c_void_p(t_idx.data_ptr()),
                  n, D, _lib.F32, _lib.I64, st)
        torch.cuda.synchronize()
        O.set_rows(src, want_tab, idx)
        assert np.array_equal(host, want_tab)
        # the host table as the cold half of a cached fetch and of an Adagrad update
        hot_ids = np.sort(rng.choice(N, 1500, replace=False)).astype(np.int64)
        t_hot_ids = dev(hot_ids)
        hot_w = dev(want_tab[hot_ids] + 1.0)
        hot_s = torch.zeros_like(hot_w)
        cold_s = torch.zeros((N, D), device="cuda")
        q = rng.integers(0, N, n).astype(np.int64)
        t_q = dev(q)
        _lib.call("hades_cached_fetch", raw, ctypes.c_void_p(hot_w.data_ptr()), ctypes.c_void_p(t_q.data_ptr()), n,
                  ctypes.c_void_p(t_hot_ids.data_ptr()), hot_ids.size, None, ctypes.c_void_p(out.data_ptr()),
                  None, D, _lib.F32, st)
        assert np.array_equal(out.cpu().numpy(), O.cached_fetch(want_tab, hot_w.cpu().numpy(), q, hot_ids))
        uq = np.unique(q)
        g = (rng.standard_normal((uq.size, D)) * 1e-3).astype(np.float32)
        t_uq, t_g = dev(uq), dev(g)
        _lib.call("hades_adagrad_update", ctypes.c_void_p(t_uq.data_ptr()), ctypes.c_void_p(t_g.data_ptr()), None,
                  uq.size, D, ctypes.c_void_p(t_hot_ids.data_ptr()), hot_ids.size, None,
                  ctypes.c_void_p(hot_w.data_ptr()), ctypes.c_void_p(hot_s.data_ptr()), raw,
                  ctypes.c_void_p(cold_s.data_ptr()), None, 0, 0.01, 1e-10, st)
        torch.cuda.synchronize()
        hw, hs, cs = (want_tab[hot_ids] + 1.0).astype(np.float32), np.zeros((1500, D), np.float32), np.zeros((N, D), np.float32)
        O.sparse_adagrad_step(want_tab, cs, hw, hs, hot_ids, uq, g, 0.01, 1e-10)
        assert np.array_equal(host, want_tab) and np.array_equal(hot_w.cpu().numpy(), hw)
        assert np.array_equal(cold_s.cpu().numpy(), cs)
        del host
        _lib.call("hades_host_free", raw)
    assert L.hades_host_free(None) == 0                   # freeing nothing is fine
    assert L.hades_host_alloc(None, 16) == 1              # null out pointer: an error code, no crash


def test_host_alloc_tensor_and_pageable_memory_is_refused(lib):
    """EmbCacheLib.host_alloc gives a host tensor the kernels accept as a cold table; cudaPin on a
    tensor that is already pinned is a no-op; a pageable tensor is refused by the shim with a
    RuntimeError before any kernel sees it.  (Registering pageable memory is exercised on the CPU
    side only, in tests/test_shm.py.)"""
    E, ops = lib
    rng = np.random.default_rng(1)
    t = E.host_alloc((3000, 64), torch.float32)
    assert not t.is_cuda and tuple(t.shape) == (3000, 64)
    t.copy_(torch.from_numpy(rng.standard_normal((3000, 64)).astype(np.float32)))
    idx = dev(rng.integers(0, 3000, 500).astype(np.int64))
    out = torch.empty((500, 64), device="cuda")
    E.cudaFetch2(t, idx, out)
    assert torch.equal(out.cpu(), t[idx.cpu()])
    E.cudaPin(t)                                           # already page-locked: nothing to do
    E.host_free(t)
    with pytest.raises(RuntimeError):
        E.host_free(torch.empty(4))
    pageable = torch.from_numpy(rng.standard_normal((1000, 16)).astype(np.float32))
    with pytest.raises(RuntimeError, match="pageable"):
        E.cudaFetch2(pageable, idx % 1000, torch.empty((500, 16), device="cuda"))
    # the process and the HIP runtime are still in working order
    assert torch.equal(ops.lookup(idx, torch.arange(3000, device="cuda")), idx)


def test_index_cache_accepts_host_tensors_like_the_reference(lib):
    """The reference calls IndexCache.lookup with CPU tensors and moves the result back
    (python/EmbCache/dist_emb.py:183-185): CPU in gives CPU out, with the device path's values."""
    from hades_amd.index_cache import IndexCache
    rng = np.random.default_rng(12)
    ic = IndexCache(4096)
    model = O.SACacheIndexModel(4096)
    ids = rng.integers(0, 100_000, 3000).astype(np.int64)
    got = ic.add(torch.from_numpy(ids))
    assert not got.is_cuda and np.array_equal(got.numpy(), model.add(ids))
    probe = rng.integers(0, 100_000, 2000).astype(np.int64)
    assert np.array_equal(ic.cudalookup(torch.from_numpy(probe)).numpy(), model.cudalookup(probe))
    got = ic.lookup(torch.from_numpy(probe))
    assert not got.is_cuda and np.array_equal(got.numpy(), model.lookup(probe))
    assert np.array_equal(ic.lookup(dev(probe)).cpu().numpy(), model.lookup(probe))     # device path
    ic.reset(torch.from_numpy(ids[:100]))
    model.reset(ids[:100])
    assert ic.get_valid_entries_num() == model.get_valid_entries_num()


@pytest.mark.parametrize("N,D,H,n,hot_frac", [
    (5000, 128, 500, 20_000, 0.9), (5000, 64, 500, 20_000, 1.0), (5000, 64, 500, 20_000, 0.0),
    (5000, 7, 0, 3000, 0.0), (300, 100, 300, 4097, 1.0),
    (70_000, 128, 9000, 257, 0.5), (70_000, 128, 9000, 256, 0.5), (70_000, 128, 9000, 1, 0.5),
    (1_000_000, 32, 100_000, 300_000, 0.9),          # several blocks either side of the class border
    (10, 4, 3, 0, 0.5),
])
@pytest.mark.parametrize("host_cold", [False, True])
def test_keyed_step_forward_and_backward(lib, N, D, H, n, hot_frac, host_cold):
    """forward_keyed / backward_keyed (one lookup per query; combine over class-ordered keys; cold
    class summed and updated first) against the oracle: fetched rows, distinct keys, sums, counts,
    class border and all four tables bit-exact in the deterministic-order mode; FAST sums within
    1e-5 per row and the same keys and counts."""
    _, ops = lib
    from hades_amd.sparse_optim import SparseAdagrad
    rng = np.random.default_rng(N + n + int(10 * hot_frac) + 1)
    cold, hot_ids, q = _split_case(rng, N, D, H, n, hot_frac)
    if n > 1000:
        q[: n // 4] = q[0]                       # a long run in one class
    t_cold = torch.from_numpy(cold.copy())
    t_cold = t_cold.pin_memory() if host_cold else t_cold.cuda()
    opt = SparseAdagrad(t_cold, torch.from_numpy(hot_ids), lr=0.01, eps=1e-10)
    opt.hot_w += 1.0
    hw = opt.hot_w.cpu().numpy().copy()
    kb = ops.key_bits_for(max(N, H, 2))
    t_q = dev(q)
    cw, cs, hs = cold.copy(), np.zeros_like(cold), np.zeros_like(hw)
    for it in range(2):
        grad = (rng.standard_normal((n, D)) * 1e-3).astype(np.float32)
        want_rows = O.cached_fetch(cw, hw, q, hot_ids)
        rows, state = opt.forward_keyed(t_q)
        assert np.array_equal(rows.cpu().numpy(), want_rows)
        if it == 0 and n:
            # the fast mode on the same plan first (it writes only the outputs, not the tables)
            plan, bufs = state
            fs, fc = ops.combine_apply_class(plan, dev(grad), 0, ops.COMBINE_FAST)
            ops.combine_apply_class(plan, dev(grad), 1, ops.COMBINE_FAST, out=(fs, fc))
            keys = O.class_ordered_keys(q, hot_ids, kb)
            wk, _, wc = O.combine_sequential(keys, grad)
            _, w64, _ = O.combine_float64(keys, grad)
            U = int(plan.num_unique.item())
            assert U == wk.size and np.array_equal(plan.uids[:U].cpu().numpy(), wk)
            assert np.array_equal(fc[:U].cpu().numpy(), wc)
            assert combine_tol_ok(fs[:U].cpu().numpy(), w64)
        ukeys, sums, cnts, nu, split = opt.backward_keyed(state, dev(grad), mode=ops.COMBINE_EXACT)
        torch.cuda.synchronize()
        wk, ws, wc, wsplit = O.keyed_step(cw, cs, hw, hs, hot_ids, q, grad, 0.01, 1e-10, kb)
        U = int(nu.item())
        assert U == wk.size and np.array_equal(ukeys[:U].cpu().numpy(), wk)
        assert np.array_equal(cnts[:U].cpu().numpy(), wc) and np.array_equal(sums[:U].cpu().numpy(), ws)
        assert split.tolist() == [int((O.lookup_sorted(q, hot_ids) < 0).sum()), wsplit]
        if U:
            ids = opt.distinct_ids_of(ukeys, nu)
            assert np.array_equal(np.sort(ids.cpu().numpy()), np.unique(q))
    assert np.array_equal(opt.cold_w.cpu().numpy(), cw) and np.array_equal(opt.cold_s.cpu().numpy(), cs)
    assert np.array_equal(opt.hot_w.cpu().numpy(), hw) and np.array_equal(opt.hot_s.cpu().numpy(), hs)


@pytest.mark.parametrize("host_cold", [False, True])
def test_keyed_backward_with_the_forward_rows(lib, host_cold):
    """backward_keyed(fetched_rows=rows): the cold update takes the old weights from the rows the
    forward pass fetched.  With untouched rows the result is that of the plain path, bit for bit;
    with rows altered on purpose the cold weights follow the altered rows (so they are what is
    read) while the hot class, which never uses them, is unaffected."""
    _, ops = lib
    from hades_amd.sparse_optim import SparseAdagrad
    rng = np.random.default_rng(4242)
    N, D, H, n = 30_000, 128, 3000, 40_000
    cold, hot_ids, q = _split_case(rng, N, D, H, n, 0.7)
    q[:500] = q[0]
    grad = (rng.standard_normal((n, D)) * 1e-3).astype(np.float32)
    kb = ops.key_bits_for(N)

    def make():
        t = torch.from_numpy(cold.copy())
        return SparseAdagrad(t.pin_memory() if host_cold else t.cuda(), torch.from_numpy(hot_ids))

    plain, reuse, altered = make(), make(), make()
    t_q, t_g = dev(q), dev(grad)
    for it in range(2):
        rows, st = plain.forward_keyed(t_q)
        plain.backward_keyed(st, t_g, mode=ops.COMBINE_EXACT, fetched_rows=None)
        assert not st[0].reused_rows
        rows2, st2 = reuse.forward_keyed(t_q)
        assert torch.equal(rows, rows2)
        reuse.backward_keyed(st2, t_g, mode=ops.COMBINE_EXACT, fetched_rows=rows2)
        torch.cuda.synchronize()
        for a, b in ((plain.cold_w, reuse.cold_w), (plain.cold_s, reuse.cold_s),
                     (plain.hot_w, reuse.hot_w), (plain.hot_s, reuse.hot_s)):
            assert torch.equal(a.cpu(), b.cpu())
    # altered rows: the oracle with the same altered rows
    cw, cs = cold.copy(), np.zeros_like(cold)
    hw, hs = cold[hot_ids].copy(), np.zeros((H, D), np.float32)
    rows3, st3 = altered.forward_keyed(t_q)
    bent = rows3 + 0.25
    altered.backward_keyed(st3, t_g, mode=ops.COMBINE_EXACT, fetched_rows=bent)
    torch.cuda.synchronize()
    O.keyed_step(cw, cs, hw, hs, hot_ids, q, grad, 0.01, 1e-10, kb, fetched_rows=bent.cpu().numpy())
    assert np.array_equal(altered.cold_w.cpu().numpy(), cw) and np.array_equal(altered.cold_s.cpu().numpy(), cs)
    assert np.array_equal(altered.hot_w.cpu().numpy(), hw) and np.array_equal(altered.hot_s.cpu().numpy(), hs)
    assert not np.array_equal(cw, plain.cold_w.cpu().numpy())


@pytest.mark.parametrize("host_cold", [False, True])
@pytest.mark.parametrize("kind", ["adagrad", "adam"])
def test_keyed_backward_reuses_the_forward_rows_only_while_the_table_is_unwritten(lib, host_cold, kind):
    """The guarded default of backward_keyed.  With nothing in between, the cold update takes its
    old weights from the forward rows and leaves the tables of the re-reading path, bit for bit.
    A second update of the same rows between the forward and the backward half, an in-place torch
    write to the cold table, an in-place change of the rows, another forward half into the same
    rows buffer, note_table_write() and reuse_fetched_rows=False each make it read the table
    again - and the result stays that of the sequence as issued (the oracle applies the steps in
    that order)."""
    _, ops = lib
    from hades_amd.sparse_optim import SparseAdagrad, SparseAdam
    rng = np.random.default_rng(777 + host_cold)
    N, D, H, n = 20_000, 64, 2000, 30_000
    cold, hot_ids, q = _split_case(rng, N, D, H, n, 0.6)
    q2 = q.copy()
    rng.shuffle(q2)
    q2[: n // 2] = rng.integers(0, N, n // 2)          # shares many cold ids with q
    g1 = (rng.standard_normal((n, D)) * 1e-3).astype(np.float32)
    g2 = (rng.standard_normal((n, D)) * 1e-3).astype(np.float32)
    t_q, t_q2, t_g1, t_g2 = dev(q), dev(q2), dev(g1), dev(g2)

    def make(**kw):
        t = torch.from_numpy(cold.copy())
        t = t.pin_memory() if host_cold else t.cuda()
        if kind == "adam":
            return SparseAdam(t, torch.from_numpy(hot_ids), **kw)
        return SparseAdagrad(t, torch.from_numpy(hot_ids), **kw)

    def tables(o):
        ts = ((o.cold_w, o.cold_s, o.hot_w, o.hot_s) if kind == "adagrad" else
              (o.cold_w, o.cold_step, o.cold_m, o.cold_v, o.hot_w, o.hot_step, o.hot_m, o.hot_v))
        torch.cuda.synchronize()
        return [t.cpu().clone() for t in ts]

    def same(a, b):
        return all(torch.equal(x, y) for x, y in zip(tables(a), tables(b)))

    guarded, reread, off = make(), make(), make(reuse_fetched_rows=False)
    # 1. nothing in between: reuse, and the tables of the re-reading path
    for it in range(2):
        _, st = guarded.forward_keyed(t_q)
        guarded.backward_keyed(st, t_g1, mode=ops.COMBINE_EXACT)
        assert st[0].reused_rows == bool(n)
        _, st_r = reread.forward_keyed(t_q)
        reread.backward_keyed(st_r, t_g1, mode=ops.COMBINE_EXACT, fetched_rows=None)
        assert not st_r[0].reused_rows
        _, st_o = off.forward_keyed(t_q)
        off.backward_keyed(st_o, t_g1, mode=ops.COMBINE_EXACT)
        assert not st_o[0].reused_rows
    assert same(guarded, reread) and same(off, reread)

    # 2. a second update of overlapping rows between the two halves: fall back, stay exact
    for o, kw in ((guarded, {}), (reread, {"fetched_rows": None})):
        _, st = o.forward_keyed(t_q)
        u2, s2, _ = ops.combine(t_q2, t_g2, mode=ops.COMBINE_EXACT)
        o.update(u2, s2)                                      # writes cold rows q also names
        o.backward_keyed(st, t_g1, mode=ops.COMBINE_EXACT, **kw)
        assert not st[0].reused_rows
    assert same(guarded, reread)
    if kind == "adagrad":                                     # and that is what the oracle says
        cw, cs = cold.copy(), np.zeros_like(cold)
        hw, hs = cold[hot_ids].copy(), np.zeros((H, D), np.float32)
        kb = ops.key_bits_for(N)
        for _ in range(2):
            O.keyed_step(cw, cs, hw, hs, hot_ids, q, g1, 0.01, 1e-10, kb)
        wu, ws, _ = O.combine_sequential(q2, g2)
        O.sparse_adagrad_step(cw, cs, hw, hs, hot_ids, wu, ws, 0.01, 1e-10)
        O.keyed_step(cw, cs, hw, hs, hot_ids, q, g1, 0.01, 1e-10, kb)
        got = tables(guarded)
        for a, b in zip(got, (cw, cs, hw, hs)):
            assert np.array_equal(a.numpy(), b)

    # 3. the other ways the rows stop standing for the table
    def backward_after(spoil):
        rows, st = guarded.forward_keyed(t_q)
        rows_r, st_r = reread.forward_keyed(t_q)
        spoil(guarded, rows)
        spoil(reread, rows_r)
        guarded.backward_keyed(st, t_g1, mode=ops.COMBINE_EXACT)
        reread.backward_keyed(st_r, t_g1, mode=ops.COMBINE_EXACT, fetched_rows=None)
        return st[0].reused_rows

    some = torch.from_numpy(np.unique(q)[:50])

    def table_write(o, rows):
        torch.cuda.synchronize()
        idx = some if not o.cold_w.is_cuda else some.cuda()
        o.cold_w[idx] += 0.5                                   # torch in place: the version counter moves

    assert not backward_after(table_write)
    assert same(guarded, reread)
    assert not backward_after(lambda o, rows: rows.mul_(2.0))  # the rows no longer hold the table's values
    assert same(guarded, reread)
    assert not backward_after(lambda o, rows: o.note_table_write())
    assert same(guarded, reread)

    def second_forward_into_the_same_buffer(o, rows):
        o.forward_keyed(t_q2, out=rows, slot=1)                # raw-pointer write: no version bump
    assert not backward_after(second_forward_into_the_same_buffer)
    assert same(guarded, reread)
    assert backward_after(lambda o, rows: None)                # and with nothing in between it reuses again
    assert same(guarded, reread)


@pytest.mark.parametrize("reuse", [True, False])
def test_keyed_step_on_an_interleaved_host_table(lib, reuse):
    """Weights and Adagrad state of the cold rows side by side in one pinned host table
    [N, 2, D] (weight_cold = t[:, 0], cold_state = t[:, 1]): forward_keyed / backward_keyed over
    the row-strided views, with and without the reuse of the forward rows, against the oracle -
    rows, distinct keys, sums and all four tables bit-exact over three steps."""
    _, ops = lib
    from hades_amd.sparse_optim import SparseAdagrad
    rng = np.random.default_rng(31 + reuse)
    N, D, H, n = 9000, 128, 900, 25_000
    cold, hot_ids, q = _split_case(rng, N, D, H, n, 0.5)
    q[:300] = q[1]
    both = torch.zeros((N, 2, D), dtype=torch.float32).pin_memory()
    both[:, 0] = torch.from_numpy(cold)
    opt = SparseAdagrad(both[:, 0], torch.from_numpy(hot_ids), lr=0.01, eps=1e-10,
                        cold_state=both[:, 1], reuse_fetched_rows=reuse)
    opt.hot_w += 1.0
    hw = opt.hot_w.cpu().numpy().copy()
    cw, cs, hs = cold.copy(), np.zeros_like(cold), np.zeros_like(hw)
    kb = ops.key_bits_for(max(N, H, 2))
    t_q = dev(q)
    for it in range(3):
        grad = (rng.standard_normal((n, D)) * 1e-3).astype(np.float32)
        rows, state = opt.forward_keyed(t_q)
        assert np.array_equal(rows.cpu().numpy(), O.cached_fetch(cw, hw, q, hot_ids))
        ukeys, sums, cnts, nu, split = opt.backward_keyed(state, dev(grad), mode=ops.COMBINE_EXACT)
        torch.cuda.synchronize()
        assert state[0].reused_rows == reuse
        wk, ws, wc, wsplit = O.keyed_step(cw, cs, hw, hs, hot_ids, q, grad, 0.01, 1e-10, kb)
        U = int(nu.item())
        assert U == wk.size and np.array_equal(ukeys[:U].cpu().numpy(), wk)
        assert np.array_equal(cnts[:U].cpu().numpy(), wc) and np.array_equal(sums[:U].cpu().numpy(), ws)
    assert np.array_equal(both[:, 0].numpy(), cw) and np.array_equal(both[:, 1].numpy(), cs)
    assert np.array_equal(opt.hot_w.cpu().numpy(), hw) and np.array_equal(opt.hot_s.cpu().numpy(), hs)


@pytest.mark.parametrize("kind", ["adagrad", "adam"])
@pytest.mark.parametrize("host_cold", [False, True])
@pytest.mark.parametrize("dim", [128, 7])
def test_cold_update_that_sums_its_own_runs(lib, kind, host_cold, dim):
    """backward_keyed's cold update adds up the gradient rows of every cold run itself (occurrence
    order, from +0.0) instead of reading a segmented sum.  Against the path with the segmented-sum
    kernels in front (fuse_cold_sums = False), in the deterministic-order mode: every table,
    the returned sums and counts bit-equal over two steps - with cold runs of 1, 2, 5, 70 and
    3 000 occurrences, gradient rows holding -0.0, and the forward rows reused or not.  In the
    fast mode the returned sums agree within the combine's tolerance."""
    _, ops = lib
    from hades_amd.sparse_optim import SparseAdagrad, SparseAdam
    rng = np.random.default_rng(5150 + dim + host_cold)
    N, H, n = 40_000, 4000, 30_000
    cold, hot_ids, q = _split_case(rng, N, dim, H, n, 0.5)
    cold_ids = np.setdiff1d(np.arange(N, dtype=np.int64), hot_ids)
    at = 0
    for k, length in enumerate((2, 5, 70, 3000)):          # planted cold runs, spread over the batch
        where = rng.choice(n, length, replace=False)
        q[where] = cold_ids[100 + k]
    grads = [(rng.standard_normal((n, dim)) * 1e-3).astype(np.float32) for _ in range(2)]
    grads[0][::7] = -0.0
    t_q = dev(q)

    def make(fuse, reuse):
        t = torch.from_numpy(cold.copy())
        t = t.pin_memory() if host_cold else t.cuda()
        cls = SparseAdam if kind == "adam" else SparseAdagrad
        o = cls(t, torch.from_numpy(hot_ids), reuse_fetched_rows=reuse)
        o.fuse_cold_sums = fuse
        return o

    def tables(o):
        ts = ((o.cold_w, o.cold_s, o.hot_w, o.hot_s) if kind == "adagrad" else
              (o.cold_w, o.cold_step, o.cold_m, o.cold_v, o.hot_w, o.hot_step, o.hot_m, o.hot_v))
        torch.cuda.synchronize()
        return [t.cpu().clone() for t in ts]

    for reuse in (True, False):
        fused, plain = make(True, reuse), make(False, reuse)
        for g in grads:
            outs = []
            for o in (fused, plain):
                _, st = o.forward_keyed(t_q)
                uk, sums, cnts, nu, split = o.backward_keyed(st, dev(g), mode=ops.COMBINE_EXACT)
                torch.cuda.synchronize()
                U = int(nu.item())
                outs.append((uk[:U].cpu(), sums[:U].cpu(), cnts[:U].cpu(), split.cpu()))
            for a, b in zip(outs[0], outs[1]):
                assert torch.equal(a, b)
            # signed zeros included: compare the bit patterns of the sums
            assert np.array_equal(outs[0][1].numpy().view(np.uint32), outs[1][1].numpy().view(np.uint32))
        for a, b in zip(tables(fused), tables(plain)):
            assert torch.equal(a, b)
    # fast mode: the returned sums of both paths within tolerance of the float64 sums
    fused = make(True, True)
    _, st = fused.forward_keyed(t_q)
    uk, sums, cnts, nu, split = fused.backward_keyed(st, dev(grads[1]), mode=ops.COMBINE_FAST)
    U = int(nu.item())
    keys = O.class_ordered_keys(q, hot_ids, ops.key_bits_for(N))
    wk, w64, wc = O.combine_float64(keys, grads[1])
    assert np.array_equal(uk[:U].cpu().numpy(), wk) and np.array_equal(cnts[:U].cpu().numpy(), wc)
    assert combine_tol_ok(sums[:U].cpu().numpy(), w64)


@pytest.mark.parametrize("kind", ["adagrad", "adam"])
@pytest.mark.parametrize("average", ["mean", "one_plus"])
@pytest.mark.parametrize("host_cold", [False, True])
def test_keyed_and_split_steps_that_average_like_the_reference(lib, kind, average, host_cold):
    """The reference's update averages duplicate ids before the row update (unique_grads,
    python/EmbCache/sparse_optim.py:142-157,613).  backward_keyed(average=...) and
    step_split(average=...) do the division on the device, inside the update kernels (keyed) or in
    place on the combined rows (split): all tables bit-equal to the oracle's combine -> division ->
    row update over three steps, with long runs in both classes and the summing cold update on
    and off."""
    _, ops = lib
    from hades_amd.sparse_optim import SparseAdagrad, SparseAdam
    rng = np.random.default_rng(303 + host_cold)
    N, D, H, n = 30_000, 64, 3000, 24_000
    cold, hot_ids, q = _split_case(rng, N, D, H, n, 0.6)
    cold_ids = np.setdiff1d(np.arange(N, dtype=np.int64), hot_ids)
    q[rng.choice(n, 700, replace=False)] = hot_ids[5]
    q[rng.choice(n, 90, replace=False)] = cold_ids[7]
    kb = ops.key_bits_for(N)
    t_q = dev(q)

    def make():
        t = torch.from_numpy(cold.copy())
        t = t.pin_memory() if host_cold else t.cuda()
        return (SparseAdam if kind == "adam" else SparseAdagrad)(t, torch.from_numpy(hot_ids))

    def tables(o):
        ts = ((o.cold_w, o.cold_s, o.hot_w, o.hot_s) if kind == "adagrad" else
              (o.cold_w, o.cold_step, o.cold_m, o.cold_v, o.hot_w, o.hot_step, o.hot_m, o.hot_v))
        torch.cuda.synchronize()
        return [t.cpu().numpy().copy() for t in ts]

    keyed, unfused, split, serial = make(), make(), make(), make()
    unfused.fuse_cold_sums = False
    if kind == "adagrad":
        want = [cold.copy(), np.zeros_like(cold), cold[hot_ids].copy(), np.zeros((H, D), np.float32)]
    else:
        z = lambda *sh: np.zeros(sh, np.float32)
        want = [cold.copy(), z(N), z(N, D), z(N, D), cold[hot_ids].copy(), z(H), z(H, D), z(H, D)]
    for it in range(3):
        g = (rng.standard_normal((n, D)) * 1e-3).astype(np.float32)
        t_g = dev(g)
        for o in (keyed, unfused):
            _, st = o.forward_keyed(t_q)
            uk, sums, cnts, nu, _ = o.backward_keyed(st, t_g, mode=ops.COMBINE_EXACT, average=average)
        split.step_split(t_q, t_g, mode=ops.COMBINE_EXACT, average=average)
        if True:
            serial.step(t_q, t_g, mode=ops.COMBINE_EXACT, average=average)      # one kernel, lookup inside
        if kind == "adagrad":
            wk, ws, wc, _ = O.keyed_step(want[0], want[1], want[2], want[3], hot_ids, q, g, 0.01, 1e-10, kb,
                                         average=average)
        else:
            wk, ws, wc, _ = O.keyed_step_adam(want[:4], want[4:], hot_ids, q, g, 0.01, 0.9, 0.999, 1e-8, kb,
                                              average=average)
        U = int(nu.item())
        # the returned rows stay the sums, the counts the occurrences
        assert np.array_equal(uk[:U].cpu().numpy(), wk) and np.array_equal(cnts[:U].cpu().numpy(), wc)
        assert np.array_equal(sums[:U].cpu().numpy(), ws)
    tk, tu, tsp, tse = tables(keyed), tables(unfused), tables(split), tables(serial)
    for a, b, c, e, w in zip(tk, tu, tsp, tse, want):
        assert np.array_equal(a, b) and np.array_equal(a, c) and np.array_equal(a, e)
        if kind == "adagrad":
            assert np.array_equal(a, w)
    if kind == "adam":      # the oracle's Adam is pinned to 1e-4 of one update only (device powf)
        for a, w in zip(tk, want):
            assert np.allclose(a, w, rtol=0, atol=5e-6)


@pytest.mark.parametrize("kind", ["adam", "adagrad"])
@pytest.mark.parametrize("pin", [True, False])
def test_dist_emb_module_trains_like_the_explicit_keyed_calls(lib, kind, pin):
    """DistEmb + the trace-driven optimizer (the reference's training loop: emb(ids) ... backward
    ... optimizer.step(), python/EmbCache/dist_emb.py:46-47,276-288, sparse_optim.py:212-238)
    against the explicit forward_keyed / backward_keyed(average="mean") calls on an identically
    initialised row optimizer: rows of every forward call and all tables after three steps are
    bit-equal.  A step with two forward calls goes through the concatenated path and matches the
    oracle's combine -> mean -> Adagrad on the concatenation."""
    _, ops = lib
    from hades_amd import dist_emb, sparse_optim
    rng = np.random.default_rng(808 + pin)
    N, D, n = 12_000, 32, 9000
    weight = torch.from_numpy((rng.standard_normal((N, D)) * 0.05).astype(np.float32))
    hotness = torch.from_numpy(rng.integers(0, 400, N))
    emb = dist_emb.DistEmb(N, D, torch.float32, "emb", cache_rate=0.2, hotness_list=hotness,
                           hot_threshold=300, weight=weight.clone(), pin_memory=pin)
    hot_ids = emb.sparse_emb.hot_ids
    assert 0 < hot_ids.numel() <= int(N * 0.2) and bool((hotness[hot_ids] >= 300).all())
    if kind == "adam":
        opt = dist_emb.SparseAdam([emb.sparse_emb], lr=0.01)
        ref = sparse_optim.SparseAdam((weight.clone().pin_memory() if pin else weight.clone().cuda()), hot_ids, lr=0.01)
    else:
        opt = dist_emb.SparseAdagrad([emb.sparse_emb], lr=0.01)
        ref = sparse_optim.SparseAdagrad((weight.clone().pin_memory() if pin else weight.clone().cuda()), hot_ids,
                                         lr=0.01)
    eng = opt._state["emb"]
    coeff = dev((rng.standard_normal((n, D)) * 1e-2).astype(np.float32))
    emb.train()
    for it in range(3):
        ids = dev(zipfish(rng, n, N))
        rows = emb(ids)
        want_rows, state = ref.forward_keyed(ids)
        assert torch.equal(rows.detach(), want_rows)
        (rows * coeff).sum().backward()
        assert len(emb.sparse_emb.trace) == 1
        opt.step()
        assert emb.sparse_emb.trace == []
        ref.backward_keyed(state, coeff, average="mean")
        torch.cuda.synchronize()
    names = (("cold_w", "cold_step", "cold_m", "cold_v", "hot_w", "hot_step", "hot_m", "hot_v") if kind == "adam"
             else ("cold_w", "cold_s", "hot_w", "hot_s"))
    for k in names:
        assert torch.equal(getattr(eng, k).cpu(), getattr(ref, k).cpu()), k
    # evaluation mode: plain rows, no trace
    emb.eval()
    probe = dev(rng.integers(0, N, 500).astype(np.int64))
    with torch.no_grad():
        got = emb(probe)
    assert emb.sparse_emb.trace == [] and not got.requires_grad
    assert np.array_equal(got.cpu().numpy(), O.cached_fetch(eng.cold_w.cpu().numpy(), eng.hot_w.cpu().numpy(),
                                                            probe.cpu().numpy(), hot_ids.numpy()))
    if kind == "adagrad":
        # two forward calls in one step: concatenated, combined, averaged, applied once
        emb.train()
        cw, cs = eng.cold_w.cpu().numpy().copy(), eng.cold_s.cpu().numpy().copy()
        hw, hs = eng.hot_w.cpu().numpy().copy(), eng.hot_s.cpu().numpy().copy()
        ids_a, ids_b = zipfish(rng, 4000, N), zipfish(rng, 3000, N)
        ca = (rng.standard_normal((4000, D)) * 1e-2).astype(np.float32)
        cb = (rng.standard_normal((3000, D)) * 1e-2).astype(np.float32)
        ra, rb = emb(dev(ids_a)), emb(dev(ids_b))
        ((ra * dev(ca)).sum() + (rb * dev(cb)).sum()).backward()
        assert len(emb.sparse_emb.trace) == 2
        opt.step()
        torch.cuda.synchronize()
        wu, ws, wc = O.combine_sequential(np.concatenate([ids_a, ids_b]), np.concatenate([ca, cb]))
        # the concatenated path sums in the fast mode: compare through the tolerance of the combine
        O.sparse_adagrad_step(cw, cs, hw, hs, hot_ids.numpy(), wu, O.averaged(ws, wc, "mean"), 0.01, 1e-10)
        for got_t, want in ((eng.cold_w, cw), (eng.cold_s, cs), (eng.hot_w, hw), (eng.hot_s, hs)):
            assert np.allclose(got_t.cpu().numpy(), want, rtol=1e-4, atol=1e-7)


def test_lookup_split_beyond_the_in_kernel_tile_sum(lib):
    """More than 4 096 tiles of queries: the per-tile counts are prefixed by a scan kernel of their
    own instead of being summed inside every compaction block.  Same lists, same slots."""
    _, ops = lib
    rng = np.random.default_rng(99)
    N, H, n = 50_000, 7_000, 2_200_001
    hot_ids = np.sort(rng.choice(N, H, replace=False)).astype(np.int64)
    q = rng.integers(0, N, n).astype(np.int64)
    hs = ops.HotSet(dev(hot_ids))
    keys = torch.empty(n, dtype=torch.int64, device="cuda")
    loc, hot_pos, cold_pos, counts = ops.lookup_split(dev(q), hs, sort_keys=keys, key_bits=16)
    w_loc, w_hp, w_cp = O.lookup_split(q, hot_ids)
    nh, nc = counts.tolist()
    assert (nh, nc) == (w_hp.size, w_cp.size)
    assert np.array_equal(loc.cpu().numpy(), w_loc)
    assert np.array_equal(hot_pos[:nh].cpu().numpy(), w_hp) and np.array_equal(cold_pos[:nc].cpu().numpy(), w_cp)
    assert np.array_equal(keys.cpu().numpy(), O.class_ordered_keys(q, hot_ids, 16))
    # the plain two-class split of the same slots (8 rounds per thread: 1 075 tiles) agrees
    _, hp2, cp2 = ops.split(loc)
    assert torch.equal(hp2, hot_pos[:nh]) and torch.equal(cp2, cold_pos[:nc])


@pytest.mark.parametrize("dim,fdt", [(1, torch.float32), (3, torch.float32), (7, torch.float64),
                                     (100, torch.float32), (128, torch.float64), (260, torch.float32)])
@pytest.mark.parametrize("host", [False, True])
def test_listed_gather_and_scatter_row_shapes(lib, dim, fdt, host):
    """hades_fetch_listed / hades_set_listed over row widths that take the 16-, 8- and 4-byte
    paths, float32 and float64, 1-D tables, device and pinned-host tables, unaligned row-strided
    views."""
    _, ops = lib
    rng = np.random.default_rng(dim)
    N, n = 3000, 2500
    width = dim + 3                                       # rows of a wider table: stride > dim
    base = torch.from_numpy(rng.standard_normal((N, width)).astype(NP_F[fdt]))
    base = base.pin_memory() if host else base.cuda()
    table = base[:, 1:1 + dim]                            # starts one element in: unaligned rows
    ref = base.cpu().numpy().copy()
    idx = rng.integers(0, N, n).astype(np.int64)
    pos = rng.permutation(n)[: n - 100].astype(np.int64)
    cnt = torch.tensor([pos.size - 7], dtype=torch.int64, device="cuda")
    out = torch.full((n, dim), -3.0, dtype=fdt, device="cuda")
    ops.fetch_listed(table, dev(idx), dev(pos), cnt, out)
    want = O.fetch_listed(ref[:, 1:1 + dim], idx, pos, pos.size - 7, np.full((n, dim), -3.0, NP_F[fdt]))
    assert np.array_equal(out.cpu().numpy(), want)
    # scatter distinct rows back
    uidx = rng.permutation(N)[:n].astype(np.int64)
    src = rng.standard_normal((n, dim)).astype(NP_F[fdt])
    ops.set_listed(dev(src), table, dev(uidx), dev(pos), cnt)
    torch.cuda.synchronize()
    view = ref[:, 1:1 + dim].copy()
    O.set_listed(src, view, uidx, pos, pos.size - 7)
    ref[:, 1:1 + dim] = view
    assert np.array_equal(base.cpu().numpy(), ref)        # the columns outside the view are untouched
    if dim == 1:                                          # the 1-D form
        flat = torch.from_numpy(rng.standard_normal(N).astype(NP_F[fdt]))
        flat = flat.pin_memory() if host else flat.cuda()
        o1 = torch.zeros(n, dtype=fdt, device="cuda")
        ops.fetch_listed(flat, dev(idx), dev(pos), cnt, o1)
        w1 = O.fetch_listed(flat.cpu().numpy(), idx, pos, pos.size - 7, np.zeros(n, NP_F[fdt]))
        assert np.array_equal(o1.cpu().numpy(), w1)


def _adam_close(got, want, k, lr=0.01):
    """tolerances of test_adam_update: weights to 1e-4 of one update, step exact, moments to rounding"""
    if got.size == 0:
        return got.shape == want.shape
    if k == 0:
        return np.abs(got - want).max() <= 1e-4 * lr
    if k == 1:
        return np.array_equal(got, want)
    return np.allclose(got, want, rtol=1e-6, atol=1e-12)


@pytest.mark.parametrize("N,D,H,n,hot_frac", [
    (5000, 128, 500, 20_000, 0.9), (5000, 64, 500, 20_000, 1.0), (5000, 64, 500, 20_000, 0.0),
    (5000, 7, 0, 3000, 0.0), (70_000, 128, 9000, 257, 0.5), (10, 4, 3, 0, 0.5),
])
@pytest.mark.parametrize("host_cold", [False, True])
def test_sparse_adam_on_the_split_and_keyed_schedules(lib, N, D, H, n, hot_frac, host_cold):
    """SparseAdam class by class (hades_adam_update_listed through step_split,
    hades_adam_update_class through forward_keyed / backward_keyed) against (1) the one-kernel
    form on the same batch, whose arithmetic is the same instruction sequence: all eight tables
    bit-equal in the deterministic-order mode, and (2) the oracle's per-class restatement of the
    reference's SparseAdam.update (python/EmbCache/sparse_optim.py:590-685) to the tolerances of
    test_adam_update."""
    _, ops = lib
    from hades_amd.sparse_optim import SparseAdam
    rng = np.random.default_rng(N + n + int(10 * hot_frac) + 7)
    cold, hot_ids, q = _split_case(rng, N, D, H, n, hot_frac)
    if n > 1000:
        q[: n // 8] = q[0]
    kb = ops.key_bits_for(max(N, H, 2))

    def make():
        t = torch.from_numpy(cold.copy())
        return SparseAdam(t.pin_memory() if host_cold else t.cuda(), torch.from_numpy(hot_ids), lr=0.01)

    one, split, keyed = make(), make(), make()
    ocold = (cold.copy(), np.zeros(N, np.float32), np.zeros_like(cold), np.zeros_like(cold))
    ohot = (cold[hot_ids].copy(), np.zeros(H, np.float32), np.zeros((H, D), np.float32),
            np.zeros((H, D), np.float32))
    t_q = dev(q)
    for it in range(3):
        grad = (rng.standard_normal((n, D)) * 1e-2).astype(np.float32)
        t_g = dev(grad)
        one.step(t_q, t_g, mode=ops.COMBINE_EXACT)
        split.step_split(t_q, t_g, mode=ops.COMBINE_EXACT)
        rows, state = keyed.forward_keyed(t_q)
        assert np.array_equal(rows.cpu().numpy(), O.cached_fetch(ocold[0], ohot[0], q, hot_ids))
        keyed.backward_keyed(state, t_g, mode=ops.COMBINE_EXACT)
        torch.cuda.synchronize()
        O.keyed_step_adam(ocold, ohot, hot_ids, q, grad, 0.01, 0.9, 0.999, 1e-8, kb)
        # the oracle's weights drift from the device's by the tolerance of each step: restart it
        # from the device's tables so that every step is checked on its own
        for k, name in enumerate(("w", "step", "m", "v")):
            for tabs, o, hot in ((ocold, one, False), (ohot, one, True)):
                got = getattr(o, ("hot_" if hot else "cold_") + name).cpu().numpy()
                assert _adam_close(got, tabs[k], k), (it, name, hot)
                tabs[k][...] = got
    for name in ("w", "step", "m", "v"):
        for pre in ("hot_", "cold_"):
            a = getattr(one, pre + name).cpu()
            assert torch.equal(a, getattr(split, pre + name).cpu()), pre + name
            assert torch.equal(a, getattr(keyed, pre + name).cpu()), pre + name


def test_sparse_adam_keyed_with_the_forward_rows(lib):
    """backward_keyed(fetched_rows=...) with SparseAdam: untouched rows give the plain result bit
    for bit; rows altered on purpose move the cold weights by exactly the alteration."""
    _, ops = lib
    from hades_amd.sparse_optim import SparseAdam
    rng = np.random.default_rng(99)
    N, D, H, n = 20_000, 64, 2000, 30_000
    cold, hot_ids, q = _split_case(rng, N, D, H, n, 0.6)
    grad = (rng.standard_normal((n, D)) * 1e-2).astype(np.float32)

    def make():
        return SparseAdam(torch.from_numpy(cold.copy()).pin_memory(), torch.from_numpy(hot_ids))

    plain, reuse, altered = make(), make(), make()
    t_q, t_g = dev(q), dev(grad)
    rows, st = plain.forward_keyed(t_q)
    plain.backward_keyed(st, t_g, mode=ops.COMBINE_EXACT)
    rows2, st2 = reuse.forward_keyed(t_q)
    reuse.backward_keyed(st2, t_g, mode=ops.COMBINE_EXACT, fetched_rows=rows2)
    rows3, st3 = altered.forward_keyed(t_q)
    altered.backward_keyed(st3, t_g, mode=ops.COMBINE_EXACT, fetched_rows=rows3 + 0.25)
    torch.cuda.synchronize()
    for name in ("w", "step", "m", "v"):
        for pre in ("hot_", "cold_"):
            assert torch.equal(getattr(plain, pre + name).cpu(), getattr(reuse, pre + name).cpu())
            if pre + name != "cold_w":
                assert torch.equal(getattr(plain, pre + name).cpu(), getattr(altered, pre + name).cpu())
    touched = np.unique(q[O.lookup_sorted(q, hot_ids) < 0])
    diff = altered.cold_w.numpy() - plain.cold_w.numpy()
    assert np.allclose(diff[touched], 0.25, atol=1e-6)
    mask = np.ones(N, bool); mask[touched] = False
    assert np.array_equal(diff[mask], np.zeros_like(diff[mask]))


@pytest.mark.parametrize("host", [False, True])
def test_fetch_listed_restricted_to_a_set(lib, host):
    """hades_fetch_listed_in_set: only positions whose table row is in the ascending set are
    fetched; every other row of the output keeps its value; set count and list count are read
    on the device; an empty set moves nothing."""
    _, ops = lib
    rng = np.random.default_rng(31)
    N, D, n = 5000, 96, 4000
    table = rng.standard_normal((N, D)).astype(np.float32)
    t = torch.from_numpy(table)
    t = t.pin_memory() if host else t.cuda()
    idx = rng.integers(0, N, n).astype(np.int64)
    pos = rng.permutation(n)[: n - 300].astype(np.int64)
    members = np.sort(rng.choice(N, 700, replace=False)).astype(np.int64)
    padded = np.concatenate([members, np.arange(N, N + 50)])       # entries past the count: ignored
    for live, set_live in ((pos.size, members.size), (pos.size - 11, 123), (pos.size, 0), (0, members.size)):
        out = torch.full((n, D), -7.0, dtype=torch.float32, device="cuda")
        ops.fetch_listed(t, dev(idx), dev(pos), torch.tensor([live], device="cuda"), out,
                         only_in=dev(padded), only_in_count=torch.tensor([set_live], device="cuda"))
        want = np.full((n, D), -7.0, np.float32)
        p = pos[:live]
        keep = p[np.isin(idx[p], members[:set_live])]
        want[keep] = table[idx[keep]]
        assert np.array_equal(out.cpu().numpy(), want)
        assert live == 0 or set_live == 0 or keep.size > 0


@pytest.mark.parametrize("N,D,H,n,hot_frac", [
    (3000, 64, 300, 5000, 0.5),             # small cold table: most cold rows of a batch were just updated
    (200_000, 128, 20_000, 60_000, 0.8),    # a few refreshed rows among many
    (5000, 32, 0, 4000, 0.0),               # no hot set
    (5000, 32, 500, 4000, 1.0),             # no cold rows
])
@pytest.mark.parametrize("host_cold", [False, True])
@pytest.mark.parametrize("kind", ["adagrad", "adam"])
def test_pipelined_keyed_steps_equal_one_batch_at_a_time(lib, N, D, H, n, hot_frac, host_cold, kind):
    """prefetch_keyed / backward_keyed(join=False) / finish_prefetch over six different batches:
    the rows every batch receives and all tables at the end equal, bit for bit, those of the same
    optimizer run one batch at a time (forward_keyed, backward_keyed) - which the tests above pin
    to the oracle - and, for Adagrad, the oracle's own sequence of keyed steps.  Both with the
    cold update reading the table and with it taking the old rows from the fetched ones."""
    _, ops = lib
    from hades_amd.sparse_optim import SparseAdagrad, SparseAdam
    rng = np.random.default_rng(N + n + 17)
    cold, hot_ids, q0 = _split_case(rng, N, D, H, n, hot_frac)
    steps = 6
    is_hot_row = np.zeros(N, bool)
    is_hot_row[hot_ids] = True
    cold_ids = np.flatnonzero(~is_hot_row).astype(np.int64)

    def draw():
        m = rng.random(n) < hot_frac
        if H == 0:
            m[:] = False
        if cold_ids.size == 0:
            m[:] = True
        hq = hot_ids[rng.integers(0, max(H, 1), n)] if H else np.zeros(n, np.int64)
        cq = cold_ids[rng.integers(0, max(cold_ids.size, 1), n)] if cold_ids.size else np.zeros(n, np.int64)
        return np.where(m, hq, cq).astype(np.int64)

    qs = [q0] + [draw() for _ in range(steps - 1)]
    grads = [(rng.standard_normal((n, D)) * 1e-2).astype(np.float32) for _ in range(steps)]
    kb = ops.key_bits_for(max(N, H, 2))

    def make():
        t = torch.from_numpy(cold.copy())
        t = t.pin_memory() if host_cold else t.cuda()
        if kind == "adam":
            return SparseAdam(t, torch.from_numpy(hot_ids))
        return SparseAdagrad(t, torch.from_numpy(hot_ids), lr=0.01, eps=1e-10)

    def tables(o):
        names = ("w", "step", "m", "v") if kind == "adam" else ("w", "s")
        return [getattr(o, pre + nm).cpu() for pre in ("cold_", "hot_") for nm in names]

    t_q = [dev(x) for x in qs]
    t_g = [dev(x) for x in grads]
    for reuse in (False, True):
        seq, pipe = make(), make()
        seq_rows = []
        for k in range(steps):
            rows, st = seq.forward_keyed(t_q[k])
            seq_rows.append(rows.clone())
            seq.backward_keyed(st, t_g[k], mode=ops.COMBINE_EXACT, fetched_rows=rows if reuse else None)
        bufs = [torch.empty((n, D), dtype=torch.float32, device="cuda") for _ in range(2)]
        rows, st = pipe.forward_keyed(t_q[0], out=bufs[0], slot=0)
        refreshed = 0
        for k in range(steps):
            assert torch.equal(rows, seq_rows[k]), (reuse, k)
            nxt = None
            if k + 1 < steps:
                nxt = pipe.prefetch_keyed(t_q[k + 1], slot=(k + 1) % 2, out=bufs[(k + 1) % 2])
            pipe.backward_keyed(st, t_g[k], mode=ops.COMBINE_EXACT, fetched_rows=rows if reuse else None,
                                join=nxt is None)
            if nxt is not None:
                prev_cold = np.unique(qs[k][~np.isin(qs[k], hot_ids)])
                refreshed += int(np.isin(qs[k + 1], prev_cold).sum())
                rows, st = pipe.finish_prefetch(nxt, after=st)
        torch.cuda.synchronize()
        for a, b in zip(tables(seq), tables(pipe)):
            assert torch.equal(a, b), reuse
        if hot_frac < 1.0:
            assert refreshed > 0            # the case does exercise the refresh
        if kind == "adagrad" and not reuse:
            cw, cs = cold.copy(), np.zeros_like(cold)
            hw, hs = cold[hot_ids].copy(), np.zeros((H, D), np.float32)
            for k in range(steps):
                assert np.array_equal(seq_rows[k].cpu().numpy(), O.cached_fetch(cw, hw, qs[k], hot_ids))
                O.keyed_step(cw, cs, hw, hs, hot_ids, qs[k], grads[k], 0.01, 1e-10, kb)
            got = tables(pipe)
            assert np.array_equal(got[0].numpy(), cw) and np.array_equal(got[1].numpy(), cs)
            assert np.array_equal(got[2].numpy(), hw) and np.array_equal(got[3].numpy(), hs)


@pytest.mark.parametrize("host", [False, True])
def test_listed_adagrad_also_returns_the_new_rows(lib, host):
    """hades_adagrad_update_listed with w_out: tables as without it (bit-equal to the oracle), and
    row p of w_out = the new weight row of position p for the listed positions, untouched elsewhere."""
    _, ops = lib
    rng = np.random.default_rng(77)
    N, D, n = 4000, 96, 3000
    w0 = rng.standard_normal((N, D)).astype(np.float32)
    s0 = np.abs(rng.standard_normal((N, D))).astype(np.float32)
    idx = rng.permutation(N)[:n].astype(np.int64)            # distinct rows
    grad = (rng.standard_normal((n, D)) * 1e-2).astype(np.float32)
    pos = rng.permutation(n)[: n - 200].astype(np.int64)
    live = pos.size - 13
    t_w = torch.from_numpy(w0.copy()); t_s = torch.from_numpy(s0.copy())
    t_w = t_w.pin_memory() if host else t_w.cuda()
    t_s = t_s.cuda()
    out = torch.full((n, D), 5.0, dtype=torch.float32, device="cuda")
    ops.adagrad_update_listed_(dev(idx), dev(grad), dev(pos), torch.tensor([live], device="cuda"),
                               t_w, t_s, 0.01, 1e-10, w_out=out)
    torch.cuda.synchronize()
    w, st = w0.copy(), s0.copy()
    O.adagrad_listed(idx, grad, pos, live, w, st, 0.01, 1e-10)
    assert np.array_equal(t_w.cpu().numpy(), w) and np.array_equal(t_s.cpu().numpy(), st)
    want = np.full((n, D), 5.0, np.float32)
    want[pos[:live]] = w[idx[pos[:live]]]
    assert np.array_equal(out.cpu().numpy(), want)


def test_pipelined_keyed_steps_with_batches_of_different_sizes(lib):
    """The pipelined calls with a different number of ids in every batch (the buffer sets are sized
    by the largest so far; an empty batch in the middle): rows and tables as one batch at a time."""
    _, ops = lib
    from hades_amd.sparse_optim import SparseAdagrad
    rng = np.random.default_rng(2024)
    N, D, H = 4000, 64, 400
    cold, hot_ids, _ = _split_case(rng, N, D, H, 10, 0.5)
    sizes = [3000, 1200, 5000, 0, 2500, 64, 5000]
    qs = [rng.integers(0, N, m).astype(np.int64) for m in sizes]
    grads = [(rng.standard_normal((m, D)) * 1e-2).astype(np.float32) for m in sizes]

    def make():
        return SparseAdagrad(torch.from_numpy(cold.copy()).pin_memory(), torch.from_numpy(hot_ids))

    seq, pipe = make(), make()
    seq_rows = []
    for q, g in zip(qs, grads):
        rows, st = seq.forward_keyed(dev(q))
        seq_rows.append(rows.clone())
        seq.backward_keyed(st, dev(g), mode=ops.COMBINE_EXACT, fetched_rows=rows)
    bufs = [torch.empty((max(sizes), D), dtype=torch.float32, device="cuda") for _ in range(2)]
    rows, st = pipe.forward_keyed(dev(qs[0]), out=bufs[0][:sizes[0]], slot=0)
    for k in range(len(sizes)):
        assert torch.equal(rows, seq_rows[k]), k
        nxt = None
        if k + 1 < len(sizes):
            nxt = pipe.prefetch_keyed(dev(qs[k + 1]), slot=(k + 1) % 2, out=bufs[(k + 1) % 2][:sizes[k + 1]])
        pipe.backward_keyed(st, dev(grads[k]), mode=ops.COMBINE_EXACT, fetched_rows=rows, join=nxt is None)
        if nxt is not None:
            rows, st = pipe.finish_prefetch(nxt, after=st)
    torch.cuda.synchronize()
    for name in ("cold_w", "cold_s", "hot_w", "hot_s"):
        assert torch.equal(getattr(seq, name).cpu(), getattr(pipe, name).cpu()), name


def test_prefetch_without_a_batch_before_it(lib):
    """prefetch_keyed + finish_prefetch(after=None) as the first call of a run gives what
    forward_keyed gives, and the backward half that follows leaves the same tables."""
    _, ops = lib
    from hades_amd.sparse_optim import SparseAdagrad
    rng = np.random.default_rng(5)
    N, D, H, n = 6000, 32, 600, 5000
    cold, hot_ids, q = _split_case(rng, N, D, H, n, 0.6)
    grad = (rng.standard_normal((n, D)) * 1e-2).astype(np.float32)
    a = SparseAdagrad(torch.from_numpy(cold.copy()).pin_memory(), torch.from_numpy(hot_ids))
    b = SparseAdagrad(torch.from_numpy(cold.copy()).pin_memory(), torch.from_numpy(hot_ids))
    rows_a, st_a = a.forward_keyed(dev(q))
    rows_b, st_b = b.finish_prefetch(b.prefetch_keyed(dev(q), slot=0))
    assert torch.equal(rows_a, rows_b)
    a.backward_keyed(st_a, dev(grad), mode=ops.COMBINE_EXACT)
    b.backward_keyed(st_b, dev(grad), mode=ops.COMBINE_EXACT, fetched_rows=rows_b)
    torch.cuda.synchronize()
    for name in ("cold_w", "cold_s", "hot_w", "hot_s"):
        assert torch.equal(getattr(a, name).cpu(), getattr(b, name).cpu()), name


def test_listed_adam_partial_count_and_strided_tables(lib):
    """hades_adam_update_listed over a position list with a device-side count, on tables whose
    rows are views of one [N, 3, D] block (weights, mem, power of a row next to each other):
    listed rows follow the oracle's adam_listed, every other row and the step counters of
    untouched rows stay as they were."""
    _, ops = lib
    rng = np.random.default_rng(88)
    N, D, n = 3000, 48, 2000
    block = (rng.standard_normal((N, 3, D)) * 0.1).astype(np.float32)
    block[:, 2] = np.abs(block[:, 2])                         # power >= 0
    step0 = rng.integers(0, 5, N).astype(np.float32)
    t_block = torch.from_numpy(block.copy()).cuda()
    t_step = torch.from_numpy(step0.copy()).cuda()
    idx = rng.permutation(N)[:n].astype(np.int64)
    grad = (rng.standard_normal((n, D)) * 1e-2).astype(np.float32)
    pos = rng.permutation(n)[: n - 300].astype(np.int64)
    live = pos.size - 21
    ops.adam_update_listed_(dev(idx), dev(grad), dev(pos), torch.tensor([live], device="cuda"),
                            (t_block[:, 0], t_step, t_block[:, 1], t_block[:, 2]), 0.01, 0.9, 0.999, 1e-8)
    torch.cuda.synchronize()
    w, m, v, st = block[:, 0].copy(), block[:, 1].copy(), block[:, 2].copy(), step0.copy()
    O.adam_listed(idx, grad, pos, live, w, st, m, v, 0.01, 0.9, 0.999, 1e-8)
    got = t_block.cpu().numpy()
    touched = np.zeros(N, bool); touched[idx[pos[:live]]] = True
    assert np.array_equal(t_step.cpu().numpy(), st)
    assert np.array_equal(got[~touched], block[~touched])
    assert np.abs(got[:, 0] - w).max() <= 1e-4 * 0.01                       # as in test_adam_update
    assert np.allclose(got[:, 1], m, rtol=1e-6, atol=1e-12) and np.allclose(got[:, 2], v, rtol=1e-6, atol=1e-12)


def test_cold_data_cache_with_padding_entries(lib):
    """Batches padded with the id -1 (the entries past a device-side length): the index cache
    and the cold-data cache answer -1 for them and evolve exactly as with the compacted batch -
    locs of the real ids, line contents, ages, slot arrays and the flushed rows."""
    _, ops = lib
    from hades_amd.cold_cache import ColdDataCache
    rng = np.random.default_rng(321)
    N, D, slots = 50_000, 32, 4096
    hotness = torch.from_numpy(rng.random(N).astype(np.float32) * 3).cuda()
    a = ColdDataCache(slots, D, hotness, cnt_threshold=4)
    b = ColdDataCache(slots, D, hotness, cnt_threshold=4)
    for it in range(6):
        m = 3000
        ids = rng.permutation(N)[:m].astype(np.int64)
        rows = rng.standard_normal((m, D)).astype(np.float32)
        grads = rng.standard_normal((m, D)).astype(np.float32)
        # the padded form: the real entries scattered over 2.5 x as many positions, -1 elsewhere
        P = 7500
        where = np.sort(rng.permutation(P)[:m])
        pid = np.full(P, -1, np.int64); pid[where] = ids
        prow = rng.standard_normal((P, D)).astype(np.float32); prow[where] = rows
        pgrad = rng.standard_normal((P, D)).astype(np.float32); pgrad[where] = grads
        la = a.accumulate_gradients_cold_remote(dev(ids), dev(grads))
        lb = b.accumulate_gradients_cold_remote(dev(pid), dev(pgrad))
        assert np.array_equal(lb.cpu().numpy()[where], la.cpu().numpy())
        assert (np.delete(lb.cpu().numpy(), where) == -1).all()
        miss = la.cpu().numpy() < 0
        ua = a.update_cache(dev(ids[miss]), dev(rows[miss]))
        pid2 = np.full(P, -1, np.int64); pid2[where[miss]] = ids[miss]
        ub = b.update_cache(dev(pid2), dev(prow))
        assert np.array_equal(ub.cpu().numpy()[where[miss]], ua.cpu().numpy())
        fa = a.staled_gradients_remote_padded(slots)
        fb = b.staled_gradients_remote_padded(slots)
        k = int(fa[3].item())
        assert k == int(fb[3].item())
        for x, y in zip(fa[:3], fb[:3]):
            assert torch.equal(x[:k], y[:k])
    torch.cuda.synchronize()
    for name in ("emb_cache_buff", "grad_cache_buff", "grad_cnt_cache_buff", "grad_idx_cache_buff"):
        assert torch.equal(getattr(a, name), getattr(b, name)), name
    assert torch.equal(a.index.line_ids, b.index.line_ids) and torch.equal(a.index.line_age, b.index.line_age)
