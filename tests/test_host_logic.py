"""Host-side logic that needs no GPU: the drop-in module's surface and argument checks, hot-set
placement, the synthetic workload generators."""
import inspect

import numpy as np
import pytest
import torch

import hades_amd
from hades_amd import cache, synth
from oracle import hades_oracle as O


def test_dropin_surface_matches_reference_binding():
    # names and argument order of src/pybind.cc:46-70
    E = hades_amd.install_as_embcachelib()
    import EmbCacheLib
    assert EmbCacheLib is E
    want = {
        "cudaSplit": ["ids", "mask"],
        "cudaPin": ["tensor"], "cudaUnpin": ["tensor"],
        "cudaFetch": ["src", "src_index", "dst", "dst_index"],
        "cudaFetch2": ["src", "src_index", "dst"],
        "cudaFetchWithCache2": ["cpu_src", "gpu_src", "src_index", "index_map", "dst"],
        "cudaSet": ["src", "dst", "dst_index"],
        "cudaSetWithCache": ["src", "cpu_dst", "gpu_dst", "dst_index", "index_map"],
        "cudaCombine": ["src", "dst", "dst_index"],
        "cudaPinPtr": ["ptr", "size"], "cudaUnpinPtr": ["ptr"],
    }
    for name, params in want.items():
        assert list(inspect.signature(getattr(E, name)).parameters) == params, name
    for name in ("cudaReminder", "cudaBinarySearch", "cudaBinarySearch2"):   # first argument is `in`
        assert callable(getattr(E, name))


def test_dropin_rejects_host_tensors_without_gpu():
    import hades_amd.EmbCacheLib as E
    a = torch.zeros((4, 4))
    i = torch.zeros(2, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="pageable host memory|device tensor"):
        E.cudaFetch2(a, i, a)
    with pytest.raises(RuntimeError):
        E.cudaSplit(i, torch.zeros(4, dtype=torch.int8))


def test_dropin_exposes_index_cache_and_later_operators_without_gpu():
    # resolved lazily (src/pybind.cc:17-45); host tensors are refused before any launch
    import hades_amd.EmbCacheLib as E
    from hades_amd import ops
    from hades_amd.index_cache import IndexCache, LocalCache
    assert E.IndexCache is IndexCache
    for name in ("get_size", "get_valid_entries_num", "get_capacity", "get_space", "add", "lookup",
                 "reset", "getall", "cudalookup"):
        assert callable(getattr(IndexCache, name)), name
    for name in ("lookup", "cudalookup", "add", "get_num_entries", "reset"):   # cache.py:18-31
        assert callable(getattr(LocalCache, name)), name
    i = torch.zeros(4, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="device tensor"):
        ops.bucket_by_owner(i, None, None, None, 4, 4)
    with pytest.raises(RuntimeError, match="int64"):
        ops.bucket_by_owner(i.to(torch.int32), None, None, None, 4, 4)
    with pytest.raises(AttributeError):
        E.no_such_function


def test_staleness_threshold_is_the_reference_formula():
    # python/EmbCache/server.py:87-88
    from hades_amd.cold_cache import staleness_threshold
    h = torch.tensor([0.0, 0.0005, 0.009, 0.099, 0.5, 1.0, 10.0])
    assert staleness_threshold(h).tolist() == [100, 100, 100, 10, 2, 1, 1]
    assert staleness_threshold(h).dtype == torch.int32


def test_select_hot_ids_matches_oracle_and_reference_recipe():
    g = torch.Generator().manual_seed(0)
    hotness = torch.rand(5000, generator=g)
    for k in (0, 1, 777, 5000):
        got = cache.select_hot_ids(hotness, k)
        assert np.array_equal(got.numpy(), O.select_hot_ids(hotness, k))
        assert got.numel() == k
        if 0 < k < 5000:
            assert hotness[got].min() >= np.sort(hotness.numpy())[-k]
    thr = cache.hot_ids_by_threshold(hotness, 0.9)
    assert np.array_equal(thr.numpy(), np.nonzero(hotness.numpy() >= 0.9)[0])


def test_rank_to_id_is_a_bijection_and_hot_ids_sorted():
    for n_rows in (10, 1000, 99_991, 2_400_000):
        ranks = torch.arange(1, n_rows + 1, dtype=torch.int64)
        ids = synth.rank_to_id(ranks, n_rows)
        assert ids.min() == 0 and ids.max() == n_rows - 1
        assert torch.unique(ids).numel() == n_rows
    hot = synth.hot_ids(99_991, 1000)
    assert bool((hot[1:] > hot[:-1]).all())
    assert set(hot.tolist()) == set(synth.rank_to_id(torch.arange(1, 1001), 99_991).tolist())


def test_zipf_sampler_statistics():
    # cfg1: 1M ranks, s = 1.1, hot = top 10 %: expected hot-hit fraction 0.919
    cfg = synth.CONFIGS["cfg1"]
    s = synth.ZipfSampler(cfg["num_rows"], cfg["zipf_s"])
    g = torch.Generator().manual_seed(1)
    ranks = s.sample_ranks(200_000, g)
    assert ranks.min() >= 1 and ranks.max() <= cfg["num_rows"]
    hit = float((ranks <= cfg["num_hot"]).float().mean())
    assert abs(hit - 0.919) < 0.005
    k = torch.arange(1, cfg["num_rows"] + 1, dtype=torch.float64)
    p1 = float(1.0 / k.pow(-1.1).sum())
    assert abs(float((ranks == 1).float().mean()) - p1) < 0.003
    ids = synth.make_ids(s, cfg["num_rows"], 65_536, 5)
    assert torch.equal(ids, synth.make_ids(s, cfg["num_rows"], 65_536, 5))      # seeded
    u = torch.unique(ids).numel()
    assert abs(u - 17_235) < 600                                                 # E[unique] of cfg1


def test_bench_refuses_more_than_one_gpu():
    import subprocess, sys, os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_key_bits_and_class_ordered_keys():
    """Host-side arithmetic of the keyed step: the bits that hold a table's ids, and the order the
    class-ordered keys induce (cold ids ascending, then hot ids ascending)."""
    from hades_amd import ops
    assert [ops.key_bits_for(n) for n in (1, 2, 3, 4, 5, 1 << 20, (1 << 20) + 1, 111_000_000, 244_000_000)] == \
        [1, 1, 2, 2, 3, 20, 21, 27, 28]
    rng = np.random.default_rng(3)
    N, H = 1000, 120
    hot = np.sort(rng.choice(N, H, replace=False)).astype(np.int64)
    q = rng.integers(0, N, 5000).astype(np.int64)
    kb = ops.key_bits_for(N)
    keys = O.class_ordered_keys(q, hot, kb)
    order = np.argsort(keys, kind="stable")
    is_hot = np.isin(q[order], hot)
    first_hot = int(np.argmax(is_hot)) if is_hot.any() else q.size
    assert not is_hot[:first_hot].any() and is_hot[first_hot:].all()
    assert np.all(np.diff(q[order][:first_hot]) >= 0) and np.all(np.diff(q[order][first_hot:]) >= 0)
    assert np.all(keys[~np.isin(q, hot)] == q[~np.isin(q, hot)])
    assert np.all((keys[np.isin(q, hot)] >> kb) == 1)


def test_split_schedule_objects_need_no_gpu_to_import():
    from hades_amd import sparse_optim
    for name in ("fetch_split", "update_split", "step_split", "forward_keyed", "backward_keyed", "join"):
        assert callable(getattr(sparse_optim.SparseAdagrad, name))


def test_bench_percentile_and_committed_traffic_summaries():
    """bench.py's percentile helper, and the HBM-traffic figures it reads from the committed
    counter summaries: every workload it nests in the default run has its kernels' lines, and
    each figure lies within a factor of two of the kernel's algorithmic bytes at that workload."""
    import bench
    assert bench.pct([3.0, 1.0, 2.0], 50) == 2.0 and bench.pct([1.0, 2.0], 50) == 1.5
    assert bench.pct([5.0], 90) == 5.0 and bench.pct([0.0, 10.0], 10) == 1.0
    t3 = bench.measured_traffic("cfg3", "fast")
    assert set(t3) >= {"hot_fetch", "seg_sum", "hot_update"}
    n_hot, u_hot, D = 923_828, 243_433, 128
    alg = {"hot_fetch": n_hot * (16 + 8 * D), "seg_sum": n_hot * (8 + 4 * D) + u_hot * 4 * D,
           "hot_update": u_hot * (8 + 20 * D)}
    for k, a in alg.items():
        assert 0.5 * a < t3[k] < 2 * a, (k, t3[k], a)
    t2 = bench.measured_traffic("cfg2", "fast")
    assert set(t2) >= {"fetch", "seg_sum", "update"}
    assert bench.measured_traffic("cfg2", "exact") == {} and bench.measured_traffic("no-such", "fast") == {}
