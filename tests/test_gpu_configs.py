"""The benchmark configurations at their full sizes on the GPU.

cfg1 is small enough for a complete comparison with the CPU oracle.  cfg3, cfg4 and cfg5 are too
large for that: they are checked through properties that need no full-size oracle run (hot rows
provably come from the HBM copy, the whole fetched batch equals plain indexing of the tables) and
through the oracle's row arithmetic on sampled ids, hot and cold, including ids whose rows lie
beyond 2^31 elements of the table.  A box without the memory skips them with the reason."""
import numpy as np
import pytest
import torch

from oracle import hades_oracle as O

pytestmark = pytest.mark.gpu


def _rows_of(table, ids):
    """rows of a (device or host) table named by a device id tensor, by plain indexing"""
    if table.is_cuda:
        return table[ids]
    return table[ids.cpu()].to(ids.device)


def _alloc_or_skip(fn, what):
    torch.cuda.empty_cache()      # blocks cached from an earlier large test go back first
    try:
        return fn()
    except (RuntimeError, MemoryError) as err:       # out of HBM / the pinned allocation is refused
        pytest.skip("%s: %s" % (what, str(err).splitlines()[0][:200]))


def test_cfg1_full_step_against_the_oracle(cuda_device):
    """1 M x 64 table, 100 K hot ids, 65 536 Zipf(1.1) ids: lookup, fetch (both schedules), combine
    (EXACT bit-exact, FAST within 1e-5 per row) and two Adagrad steps bit-exact."""
    from hades_amd import ops, synth
    from hades_amd.sparse_optim import SparseAdagrad
    cfg = synth.CONFIGS["cfg1"]
    N, D, H, n = cfg["num_rows"], cfg["dim"], cfg["num_hot"], cfg["batch"]
    table = torch.empty((N, D), dtype=torch.float32)
    synth.fill_normal_(table, 0.01, 1235)
    hot_ids = synth.hot_ids(N, H)
    sampler = synth.ZipfSampler(N, cfg["zipf_s"])
    opt = SparseAdagrad(table.cuda(), hot_ids, lr=0.01, eps=1e-10)
    opt.hot_w += 0.5                       # hot copies differ from the cold copies: sources show
    cw, cs = table.numpy().copy(), np.zeros((N, D), np.float32)
    hw, hs = opt.hot_w.cpu().numpy().copy(), np.zeros((H, D), np.float32)
    hot_np = hot_ids.numpy()
    for step in range(2):
        q = synth.make_ids(sampler, N, n, 1235_000 + step)
        g = synth.make_grads(n, D, 1235_500 + step)
        t_q, t_g = q.cuda(), g.cuda()
        assert np.array_equal(ops.lookup(t_q, opt.hot_set).cpu().numpy(), O.lookup_sorted(q.numpy(), hot_np))
        want_rows = O.cached_fetch(cw, hw, q.numpy(), hot_np)
        assert np.array_equal(opt.fetch(t_q).cpu().numpy(), want_rows)
        assert np.array_equal(opt.fetch_split(t_q).cpu().numpy(), want_rows)
        wu, ws, wc = O.combine_sequential(q.numpy(), g.numpy())
        _, w64, _ = O.combine_float64(q.numpy(), g.numpy())
        fu, fs, fc = ops.combine(t_q, t_g, N, ops.COMBINE_FAST)
        assert np.array_equal(fu.cpu().numpy(), wu) and np.array_equal(fc.cpu().numpy(), wc)
        err = np.abs(fs.cpu().numpy().astype(np.float64) - w64).max(axis=1)
        assert np.all(err <= 1e-5 * np.abs(w64).max(axis=1))          # 1e-5 relative, per row
        if step == 0:
            uids, sums, cnts, nu = opt.step(t_q, t_g, mode=ops.COMBINE_EXACT)
        else:
            uids, sums, cnts, nu = opt.step_split(t_q, t_g, mode=ops.COMBINE_EXACT)
        U = int(nu.item())
        assert U == wu.size and np.array_equal(uids[:U].cpu().numpy(), wu)
        assert np.array_equal(cnts[:U].cpu().numpy(), wc) and np.array_equal(sums[:U].cpu().numpy(), ws)
        O.sparse_adagrad_step(cw, cs, hw, hs, hot_np, wu, ws, 0.01, 1e-10)
    torch.cuda.synchronize()
    assert np.array_equal(opt.cold_w.cpu().numpy(), cw) and np.array_equal(opt.cold_s.cpu().numpy(), cs)
    assert np.array_equal(opt.hot_w.cpu().numpy(), hw) and np.array_equal(opt.hot_s.cpu().numpy(), hs)


def _sampled_update_check(opt, uids, sums, U, before, sample_ids):
    """rows of the sampled ids after the step against O.adagrad_rows on their rows before it"""
    pos = torch.searchsorted(uids[:U], sample_ids)
    assert torch.equal(uids[:U][pos], sample_ids)
    g = sums[:U][pos].cpu().numpy()
    w0, s0 = before
    w1, s1 = O.adagrad_rows(w0, s0, g, 0.01, 1e-10)
    return w1, s1


def _table_rows(opt, ids):
    """(w rows, s rows) of the ids as the optimizer holds them: hot copy if hot, else cold table;
    gathered with torch indexing only."""
    hot = opt.hot_ids
    if hot.numel():
        p = torch.searchsorted(hot, ids, right=True)
        hit = (p > 0) & (hot[(p - 1).clamp(min=0)] == ids)
    else:
        p = torch.zeros_like(ids)
        hit = torch.zeros_like(ids, dtype=torch.bool)
    w = torch.empty((ids.numel(), opt.dim), device=ids.device)
    s = torch.empty_like(w)
    if bool(hit.any()):
        w[hit], s[hit] = opt.hot_w[(p - 1)[hit]], opt.hot_s[(p - 1)[hit]]
    miss = ~hit
    if bool(miss.any()):
        w[miss], s[miss] = _rows_of(opt.cold_w, ids[miss]), _rows_of(opt.cold_s, ids[miss])
    return w.cpu().numpy(), s.cpu().numpy(), hit


@pytest.mark.parametrize("schedule", ["split", "serial"])
def test_cfg3_full_size_fetch_and_update(cuda_device, schedule):
    """111 M x 128 table: 11.1 M hot rows in HBM, the full table in pinned host memory, 1 M
    Zipf(1.05) ids.  The hot copies are shifted by one, so a hot row that came from the host table
    would show; the whole fetched batch must equal plain indexing of the two tables; after one
    step the weight and state rows of 6 000 sampled distinct ids (hot, cold, and the largest ids,
    whose rows start beyond 2^31 elements) must equal the oracle's Adagrad on their old rows."""
    from hades_amd import ops, synth
    from hades_amd.sparse_optim import SparseAdagrad
    cfg = synth.CONFIGS["cfg3"]
    N, D, H, n = cfg["num_rows"], cfg["dim"], cfg["num_hot"], cfg["batch"]
    dev = cuda_device
    table = _alloc_or_skip(lambda: torch.empty((N, D), dtype=torch.float32, pin_memory=True),
                           "cfg3 needs a 56.8 GB page-locked table")
    synth.fill_normal_(table, 0.01, 1237)
    hot_ids = synth.hot_ids(N, H, dev)
    opt = _alloc_or_skip(lambda: SparseAdagrad(table, hot_ids, lr=0.01, eps=1e-10, device=dev,
                                               state_on_device=True), "cfg3 needs 70 GB of HBM")
    opt.hot_w += 1.0
    sampler = synth.ZipfSampler(N, cfg["zipf_s"], dev)
    q = synth.make_ids(sampler, N, n, 1237_000)
    del sampler
    g = synth.make_grads(n, D, 1237_500, dev)
    # fetch: the whole batch against plain indexing
    p = torch.searchsorted(hot_ids, q, right=True)
    hit = (p > 0) & (hot_ids[(p - 1).clamp(min=0)] == q)
    assert 0.85 < float(hit.float().mean()) < 0.97
    want = _rows_of(table, q)
    want[hit] += 1.0
    got = opt.fetch_split(q) if schedule == "split" else opt.fetch(q)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    del got, want
    # sampled distinct ids: hot, cold, and the largest of the batch
    uq = torch.unique(q)
    assert int(uq[-1]) * D > 2**31
    gen = torch.Generator().manual_seed(5)
    pick = torch.randperm(uq.numel(), generator=gen)[:5000].to(dev)
    sample = torch.unique(torch.cat([uq[pick], uq[-1000:]]))
    w0, s0, s_hit = _table_rows(opt, sample)
    assert 0 < int(s_hit.sum()) < sample.numel()                      # both classes are in the sample
    if schedule == "split":
        uids, sums, cnts, nu = opt.step_split(q, g, mode=ops.COMBINE_EXACT)
    else:
        uids, sums, cnts, nu = opt.step(q, g, mode=ops.COMBINE_EXACT)
    torch.cuda.synchronize()
    U = int(nu.item())
    assert U == uq.numel() and torch.equal(uids[:U], uq)
    assert int(cnts[:U].sum()) == n
    w1, s1 = _sampled_update_check(opt, uids, sums, U, (w0, s0), sample)
    gw, gs, _ = _table_rows(opt, sample)
    assert np.array_equal(gw, w1) and np.array_equal(gs, s1)
    # rows that were not in the batch did not move
    others = torch.randint(0, N, (4000,), generator=gen).to(dev)
    others = others[~torch.isin(others, uq)]
    ow, os_, o_hit = _table_rows(opt, others)
    base = _rows_of(table, others).cpu().numpy()
    base[o_hit.cpu().numpy()] += 1.0
    assert np.array_equal(ow, base) and not os_.any()


def test_cfg3_full_size_keyed_and_pipelined(cuda_device):
    """cfg3 at full size on the schedules the benchmark times: batch A through forward_keyed;
    batch B prefetched on the side streams while A's backward half runs (its cold update takes
    the old rows from the fetched ones); B's rows completed by finish_prefetch.  A's rows equal
    plain indexing of the tables before the step; the weight and state rows of sampled distinct
    ids of A (hot, cold, ids beyond 2^31 elements) equal the oracle's Adagrad on their old rows
    and summed gradients; B's whole batch of rows equals plain indexing of the tables AFTER A's
    update - among them the cold rows that A's update wrote while B's gather was under way."""
    from hades_amd import ops, synth
    from hades_amd.sparse_optim import SparseAdagrad
    cfg = synth.CONFIGS["cfg3"]
    N, D, H, n = cfg["num_rows"], cfg["dim"], cfg["num_hot"], cfg["batch"]
    dev = cuda_device
    table = _alloc_or_skip(lambda: torch.empty((N, D), dtype=torch.float32, pin_memory=True),
                           "cfg3 needs a 56.8 GB page-locked table")
    synth.fill_normal_(table, 0.01, 1237)
    hot_ids = synth.hot_ids(N, H, dev)
    opt = _alloc_or_skip(lambda: SparseAdagrad(table, hot_ids, lr=0.01, eps=1e-10, device=dev,
                                               state_on_device=True), "cfg3 needs 70 GB of HBM")
    opt.hot_w += 1.0
    sampler = synth.ZipfSampler(N, cfg["zipf_s"], dev)
    qa = synth.make_ids(sampler, N, n, 1237_000)
    qb = synth.make_ids(sampler, N, n, 1237_001)
    del sampler
    # make sure B asks for cold rows that A updates: a few thousand of A's cold ids go into B
    pa = torch.searchsorted(hot_ids, qa, right=True)
    a_cold = qa[~((pa > 0) & (hot_ids[(pa - 1).clamp(min=0)] == qa))]
    qb[:3000] = a_cold[:3000]
    g = synth.make_grads(n, D, 1237_500, dev)

    def plain_rows(q):
        p = torch.searchsorted(hot_ids, q, right=True)
        hit = (p > 0) & (hot_ids[(p - 1).clamp(min=0)] == q)
        want = _rows_of(opt.cold_w, q)
        want[hit] = opt.hot_w[(p - 1)[hit]]
        return want

    want_a = plain_rows(qa)
    uq = torch.unique(qa)
    gen = torch.Generator().manual_seed(7)
    pick = torch.randperm(uq.numel(), generator=gen)[:5000].to(dev)
    sample = torch.unique(torch.cat([uq[pick], uq[-1000:], a_cold[:500]]))
    w0, s0, s_hit = _table_rows(opt, sample)
    assert 0 < int(s_hit.sum()) < sample.numel()
    rows_a, st_a = opt.forward_keyed(qa, slot=0)
    torch.cuda.synchronize()
    assert torch.equal(rows_a, want_a)
    del want_a
    nxt = opt.prefetch_keyed(qb, slot=1)
    ukeys, sums, cnts, nu, split = opt.backward_keyed(st_a, g, mode=ops.COMBINE_EXACT,
                                                      fetched_rows=rows_a, join=False)
    rows_b, st_b = opt.finish_prefetch(nxt, after=st_a)
    torch.cuda.synchronize()
    U = int(nu.item())
    assert U == uq.numel() and int(cnts[:U].sum()) == n
    ids = opt.distinct_ids_of(ukeys, nu)
    order = torch.argsort(ids)
    assert torch.equal(ids[order], uq)
    w1, s1 = _sampled_update_check(opt, ids[order], sums[:U][order], U, (w0, s0), sample)
    gw, gs, _ = _table_rows(opt, sample)
    assert np.array_equal(gw, w1) and np.array_equal(gs, s1)
    assert torch.equal(rows_b, plain_rows(qb))


def test_cfg3_batch_with_cold_state_in_host_memory(cuda_device):
    """The contract layout of the cold class at the size one page-locked allocation allows:
    weights and Adagrad state of the cold rows both in pinned host memory, the two rows of an id
    side by side in one [N, 2, D] table of 55.5 M ids (56.8 GB), 5.55 M hot ids in HBM, cfg3's
    batch of 1 M Zipf(1.05) ids.  Keyed schedule, two steps on the same batch (the second one
    sees non-zero state in host memory): fetched rows equal plain indexing; weight and state rows
    of sampled distinct ids (hot, cold, rows beyond 2^31 elements) equal the oracle's Adagrad on
    their old rows; the state rows of ids outside the batch stay zero."""
    from hades_amd import ops, synth
    from hades_amd.sparse_optim import SparseAdagrad
    cfg = synth.CONFIGS["cfg3"]
    N, D, H, n = cfg["num_rows"] // 2, cfg["dim"], cfg["num_hot"] // 2, cfg["batch"]
    dev = cuda_device
    both = _alloc_or_skip(lambda: torch.empty((N, 2, D), dtype=torch.float32, pin_memory=True),
                          "the interleaved table needs a 56.8 GB page-locked allocation")
    synth.fill_interleaved_(both, 0.01, 1239)
    hot_ids = synth.hot_ids(N, H, dev)
    opt = _alloc_or_skip(lambda: SparseAdagrad(both[:, 0], hot_ids, lr=0.01, eps=1e-10, device=dev,
                                               cold_state=both[:, 1]), "needs 10 GB of HBM")
    assert not opt.cold_s.is_cuda and opt.cold_s.data_ptr() == opt.cold_w.data_ptr() + 4 * D
    opt.hot_w += 1.0
    sampler = synth.ZipfSampler(N, cfg["zipf_s"], dev)
    q = synth.make_ids(sampler, N, n, 1239_000)
    del sampler
    uq = torch.unique(q)
    assert int(uq[-1]) * 2 * D > 2**31
    gen = torch.Generator().manual_seed(9)
    pick = torch.randperm(uq.numel(), generator=gen)[:5000].to(dev)
    sample = torch.unique(torch.cat([uq[pick], uq[-1000:]]))

    def plain_rows(ids):
        p = torch.searchsorted(hot_ids, ids, right=True)
        hit = (p > 0) & (hot_ids[(p - 1).clamp(min=0)] == ids)
        want = _rows_of(opt.cold_w, ids)
        want[hit] = opt.hot_w[(p - 1)[hit]]
        return want

    for step in range(2):
        g = synth.make_grads(n, D, 1239_500 + step, dev)
        w0, s0, s_hit = _table_rows(opt, sample)
        assert 0 < int(s_hit.sum()) < sample.numel()
        want = plain_rows(q)
        rows, st = opt.forward_keyed(q)
        torch.cuda.synchronize()
        assert torch.equal(rows, want)
        del want
        ukeys, sums, cnts, nu, split = opt.backward_keyed(st, g, mode=ops.COMBINE_EXACT)
        torch.cuda.synchronize()
        assert st[0].reused_rows
        U = int(nu.item())
        assert U == uq.numel() and int(cnts[:U].sum()) == n
        ids = opt.distinct_ids_of(ukeys, nu)
        order = torch.argsort(ids)
        assert torch.equal(ids[order], uq)
        w1, s1 = _sampled_update_check(opt, ids[order], sums[:U][order], U, (w0, s0), sample)
        gw, gs, _ = _table_rows(opt, sample)
        assert np.array_equal(gw, w1) and np.array_equal(gs, s1)
        assert step == 0 or s0.any()
    others = torch.randint(0, N, (4000,), generator=gen).to(dev)
    others = others[~torch.isin(others, uq)]
    _, os_, _ = _table_rows(opt, others)
    assert not os_.any()


def test_cfg5_full_size_local_aggregation_and_update(cuda_device):
    """Four 256 K batches over a 244 M x 64 table in HBM (62.5 GB plus as much Adagrad state):
    combine of the concatenation, then the update; sampled rows against the oracle, the rest of a
    sample untouched."""
    from hades_amd import ops, synth
    from hades_amd.sparse_optim import SparseAdagrad
    cfg = synth.CONFIGS["cfg5"]
    N, D, n, T = cfg["num_rows"], cfg["dim"], cfg["batch"], cfg["trainers"]
    dev = cuda_device
    table = _alloc_or_skip(lambda: torch.empty((N, D), dtype=torch.float32, device=dev),
                           "cfg5 needs a 62.5 GB table in HBM")
    synth.fill_normal_(table, 0.01, 1239)
    opt = _alloc_or_skip(lambda: SparseAdagrad(table, torch.empty(0, dtype=torch.int64), lr=0.01,
                                               eps=1e-10, device=dev), "cfg5 needs 125 GB of HBM")
    sampler = synth.ZipfSampler(N, cfg["zipf_s"], dev)
    q = torch.cat([synth.make_ids(sampler, N, n, 1239_000 + t) for t in range(T)]).contiguous()
    del sampler
    g = synth.make_grads(n * T, D, 1239_500, dev)
    uq = torch.unique(q)
    gen = torch.Generator().manual_seed(6)
    pick = torch.randperm(uq.numel(), generator=gen)[:5000].to(dev)
    sample = torch.unique(torch.cat([uq[pick], uq[-500:], uq[:500]]))
    w0, s0 = table[sample].cpu().numpy(), opt.cold_s[sample].cpu().numpy()
    uids, sums, cnts, nu = opt.step(q, g, mode=ops.COMBINE_EXACT)
    torch.cuda.synchronize()
    U = int(nu.item())
    assert U == uq.numel() and torch.equal(uids[:U], uq) and int(cnts[:U].sum()) == n * T
    # the summed rows of the sample against a sequential float32 sum on the host
    pos = torch.searchsorted(uids[:U], sample)
    few = sample[:300]
    mask = torch.isin(q, few)
    wu, ws, _ = O.combine_sequential(q[mask].cpu().numpy(), g[mask].cpu().numpy())
    assert np.array_equal(wu, few.cpu().numpy()) and np.array_equal(sums[:U][pos[:300]].cpu().numpy(), ws)
    w1, s1 = _sampled_update_check(opt, uids, sums, U, (w0, s0), sample)
    assert np.array_equal(table[sample].cpu().numpy(), w1)
    assert np.array_equal(opt.cold_s[sample].cpu().numpy(), s1)
    others = torch.randint(0, N, (4000,), generator=gen).to(dev)
    others = others[~torch.isin(others, uq)]
    assert not bool(opt.cold_s[others].any())


def test_cfg4_write_back_into_the_pinned_host_table(cuda_device):
    """512 K cold ids per step into the 4 M-slot accumulator, flushed after 8 steps and applied by
    Adagrad to the 111 M x 128 pinned-host table: sampled rows of that table after the write-back
    against the oracle (per-step sequential sums added in step order, then adagrad_rows)."""
    from hades_amd import ops, synth
    cfg = synth.CONFIGS["cfg4"]
    N, D, H, n = cfg["num_rows"], cfg["dim"], cfg["num_hot"], cfg["batch"]
    slots, every = cfg["num_slots"], cfg["flush_every"]
    dev = cuda_device
    table = _alloc_or_skip(lambda: torch.empty((N, D), dtype=torch.float32, pin_memory=True),
                           "cfg4 needs a 56.8 GB page-locked table")
    synth.fill_normal_(table, 0.01, 1238)
    cold_s = _alloc_or_skip(lambda: torch.zeros((N, D), dtype=torch.float32, device=dev),
                            "cfg4 needs 60 GB of HBM")
    sampler = synth.ZipfSampler(N - H, cfg["zipf_s"], dev)
    ids = [synth.make_ids(sampler, N, n, 1238_000 + b, rank_offset=H) for b in range(every)]
    del sampler
    grads = [synth.make_grads(n, D, 1238_500 + b, dev) for b in range(every)]
    all_ids = torch.unique(torch.cat(ids))
    gen = torch.Generator().manual_seed(7)
    pick = torch.randperm(all_ids.numel(), generator=gen)[:1500].to(dev)
    sample = torch.unique(torch.cat([all_ids[pick], all_ids[-250:], all_ids[:250]]))
    w0 = _rows_of(table, sample).cpu().numpy()
    acc = ops.ColdGradAccumulator(slots, D, id_bound=N, device=dev)
    want = np.zeros((sample.numel(), D), np.float32)
    seen = np.zeros(sample.numel(), bool)
    s_np = sample.cpu().numpy()
    for b in range(every):
        u, s, c = ops.combine(ids[b], grads[b], id_bound=N, mode=ops.COMBINE_EXACT)
        acc.accumulate(u, s, c)
        mask = torch.isin(ids[b], sample)
        wu, ws, _ = O.combine_sequential(ids[b][mask].cpu().numpy(), grads[b][mask].cpu().numpy())
        at = np.searchsorted(s_np, wu)
        want[at] = want[at] + ws                   # one float32 add per step, in step order
        seen[at] = True
    assert seen.all()
    f_ids, f_sums, f_cnts = acc.flush()
    assert torch.equal(f_ids, all_ids) and int(f_cnts.sum()) == n * every
    pos = torch.searchsorted(f_ids, sample)
    assert np.array_equal(f_sums[pos].cpu().numpy(), want)
    ops.adagrad_update_(f_ids, f_sums, None, None, table, cold_s, None, 0.01, 1e-10)
    torch.cuda.synchronize()
    w1, s1 = O.adagrad_rows(w0, np.zeros_like(w0), want, 0.01, 1e-10)
    assert np.array_equal(_rows_of(table, sample).cpu().numpy(), w1)
    assert np.array_equal(cold_s[sample].cpu().numpy(), s1)
    # the table is empty again, and rows that never got a gradient did not move
    assert acc.flush()[0].numel() == 0
