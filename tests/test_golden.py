"""The committed vectors of tests/golden/vectors.npz (made by tests/golden/make_vectors.py with
library routines and brute force only) against the CPU oracle (no GPU needed) and against the HIP
library through its C ABI (gpu marker).  Integer, index and payload results are compared
bit-exactly; fp32 sums in FAST mode within 1e-5 of the fp64 sums; Adagrad within 1e-5 relative of
torch.optim.Adagrad; Adam within 2e-4 of one update
(the reference forms 1 - beta^t in fp32, torch.optim.Adam in double)."""
import os

import numpy as np
import pytest
import torch

from oracle import hades_oracle as O

VEC = np.load(os.path.join(os.path.dirname(__file__), "golden", "vectors.npz"), allow_pickle=False)


def _eq(a, b):
    a, b = np.asarray(a), np.asarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and np.array_equal(a, b)


# ---------------------------------------------------------------------------- oracle vs vectors
def test_oracle_lookup_golden():
    assert _eq(O.lookup_sorted(VEC["lookup_q"], VEC["lookup_hot"]), VEC["lookup_loc"])


def test_oracle_split_golden():
    masks, pos = O.split3_compact(VEC["split_ids"], VEC["split_table"])
    for k in range(3):
        assert _eq(pos[k], VEC["split_pos%d" % k])
        assert _eq(VEC["split_ids"][masks[k]], VEC["split_ids%d" % k])


def test_oracle_rows_golden():
    dst = O.cached_fetch(VEC["rows_cold"], VEC["rows_hot_rows"], VEC["rows_q"], VEC["rows_hot"])
    assert _eq(dst, VEC["rows_fetch_dst"])
    cold, hot = VEC["rows_cold"].copy(), VEC["rows_hot_rows"].copy()
    O.cached_set(VEC["rows_set_src"], cold, hot, VEC["rows_set_q"], VEC["rows_hot"])
    assert _eq(cold, VEC["rows_set_cold_after"]) and _eq(hot, VEC["rows_set_hot_after"])


def test_oracle_combine_golden():
    uids, sums, cnts = O.combine_sequential(VEC["comb_idx"], VEC["comb_grad"])
    assert _eq(uids, VEC["comb_uids"]) and _eq(cnts, VEC["comb_cnts"])
    assert _eq(sums, VEC["comb_sums_seq32"])
    tu, ts, tc = O.only_unique_grads(torch.from_numpy(VEC["comb_idx"]), torch.from_numpy(VEC["comb_grad"]))
    assert _eq(tu.numpy(), VEC["comb_uids"]) and _eq(tc.numpy(), VEC["comb_cnts"])
    assert np.abs(ts.numpy() - VEC["comb_sums_f64"]).max() <= 1e-5


def _adagrad_close(w, s):
    """torch.optim.Adagrad rounds lr * (g / std), the row update here (lr * g) / std, and its
    addcmul may fuse g*g into the add: one rounding apart, so 1e-5 relative on w and 1e-6 on s
    (the HIP kernel is bit-exact against the oracle in the parity tests)."""
    assert np.allclose(w, VEC["ada_w"], rtol=1e-5, atol=1e-8)
    assert np.allclose(s, VEC["ada_s"], rtol=1e-6, atol=0)


def test_oracle_adagrad_golden():
    w, s = VEC["ada_w0"].copy(), np.zeros_like(VEC["ada_w0"])
    for g in VEC["ada_g"]:
        w, s = O.adagrad_rows(w, s, g, 0.01, 1e-10)
    _adagrad_close(w, s)


def test_oracle_adam_golden():
    w = VEC["adam_w0"].copy()
    step = np.zeros(w.shape[0], np.float32)
    m, v = np.zeros_like(w), np.zeros_like(w)
    for g in VEC["adam_g"]:
        w, step, m, v = O.adam_rows(w, step, m, v, g, 0.01, 0.9, 0.999, 1e-8)
    assert np.abs(m - VEC["adam_m"]).max() <= 1e-9 and np.abs(v - VEC["adam_v"]).max() <= 1e-12
    assert np.abs(w - VEC["adam_w"]).max() <= 2e-4 * 0.01 * len(VEC["adam_g"])


def test_oracle_accumulator_golden():
    model = O.ColdGradAccumulatorModel(VEC["acc_g0"].shape[1])
    for b in range(3):
        model.accumulate(VEC["acc_ids%d" % b], VEC["acc_g%d" % b], VEC["acc_c%d" % b])
    ids, sums, cnts = model.flush()
    assert _eq(ids, VEC["acc_flush_ids"]) and _eq(cnts, VEC["acc_flush_cnts"])
    assert _eq(sums, VEC["acc_flush_sums"])


def _keyed_close(cw, cs, hw, hs):
    """as _adagrad_close: torch.optim.Adagrad is one rounding apart from the row arithmetic"""
    assert np.allclose(cw, VEC["ss_cold_after"], rtol=1e-5, atol=1e-8)
    assert np.allclose(hw, VEC["ss_hot_after"], rtol=1e-5, atol=1e-8)
    assert np.allclose(cs, VEC["ss_cold_state"], rtol=1e-6, atol=0)
    assert np.allclose(hs, VEC["ss_hot_state"], rtol=1e-6, atol=0)


def test_oracle_split_schedule_golden():
    hot, q, kb = VEC["ss_hot"], VEC["ss_q"], int(VEC["ss_key_bits"][0])
    loc, hot_pos, cold_pos = O.lookup_split(q, hot)
    assert _eq(loc, VEC["ss_loc"]) and _eq(hot_pos, VEC["ss_hot_pos"]) and _eq(cold_pos, VEC["ss_cold_pos"])
    assert _eq(O.class_ordered_keys(q, hot, kb), VEC["ss_keys"])
    cw, cs = VEC["ss_cold"].copy(), np.zeros_like(VEC["ss_cold"])
    hw, hs = VEC["ss_hot_rows"].copy(), np.zeros_like(VEC["ss_hot_rows"])
    ukeys, sums, cnts, split = O.keyed_step(cw, cs, hw, hs, hot, q, VEC["ss_grad"], 0.01, 1e-10, kb)
    assert _eq(ukeys, VEC["ss_ukeys"]) and _eq(sums, VEC["ss_usums"]) and _eq(cnts, VEC["ss_ucnts"])
    assert split == int(VEC["ss_class_split"][1])
    _keyed_close(cw, cs, hw, hs)
    # the fetch, class by class
    want = np.stack([VEC["ss_hot_rows"][l] if l >= 0 else VEC["ss_cold"][x] for l, x in zip(VEC["ss_loc"], q)])
    assert _eq(O.fetch_split(VEC["ss_cold"], VEC["ss_hot_rows"], q, hot), want)


# ------------------------------------------------------------------------ HIP library vs vectors
def _d(name, dev):
    return torch.from_numpy(VEC[name].copy()).to(dev)


@pytest.mark.gpu
@pytest.mark.parametrize("indexed", [False, True])
def test_hip_lookup_golden(cuda_device, indexed):
    from hades_amd import ops
    hot = ops.HotSet(_d("lookup_hot", cuda_device), build_index=indexed)
    loc = ops.lookup(_d("lookup_q", cuda_device), hot)
    assert _eq(loc.cpu().numpy(), VEC["lookup_loc"])


@pytest.mark.gpu
def test_hip_split_golden(cuda_device):
    from hades_amd import ops
    ids = _d("split_ids", cuda_device)
    masks, pos, counts = ops.split3_padded(ids, _d("split_table", cuda_device).to(torch.int8))
    counts = counts.cpu().tolist()
    for k in range(3):
        want = VEC["split_pos%d" % k]
        assert counts[k] == want.size
        assert _eq(pos[k][:counts[k]].cpu().numpy(), want)
        assert _eq(ids[masks[k]].cpu().numpy(), VEC["split_ids%d" % k])


@pytest.mark.gpu
@pytest.mark.parametrize("indexed", [False, True])
def test_hip_rows_golden(cuda_device, indexed):
    from hades_amd import ops
    hot_set = ops.HotSet(_d("rows_hot", cuda_device), build_index=indexed)
    cold, hot = _d("rows_cold", cuda_device), _d("rows_hot_rows", cuda_device)
    dst = ops.cached_fetch(cold, hot, _d("rows_q", cuda_device), hot_set)
    assert _eq(dst.cpu().numpy(), VEC["rows_fetch_dst"])
    ops.cached_set(_d("rows_set_src", cuda_device), cold, hot, _d("rows_set_q", cuda_device), hot_set)
    assert _eq(cold.cpu().numpy(), VEC["rows_set_cold_after"])
    assert _eq(hot.cpu().numpy(), VEC["rows_set_hot_after"])


@pytest.mark.gpu
def test_hip_combine_golden(cuda_device):
    from hades_amd import ops
    idx, grad = _d("comb_idx", cuda_device), _d("comb_grad", cuda_device)
    for id_bound in (0, 1 << 20):
        uids, sums, cnts = ops.combine(idx, grad, id_bound=id_bound, mode=ops.COMBINE_EXACT)
        assert _eq(uids.cpu().numpy(), VEC["comb_uids"]) and _eq(cnts.cpu().numpy(), VEC["comb_cnts"])
        assert _eq(sums.cpu().numpy(), VEC["comb_sums_seq32"])
        uids, sums, cnts = ops.combine(idx, grad, id_bound=id_bound, mode=ops.COMBINE_FAST)
        assert _eq(uids.cpu().numpy(), VEC["comb_uids"]) and _eq(cnts.cpu().numpy(), VEC["comb_cnts"])
        assert np.abs(sums.cpu().numpy() - VEC["comb_sums_f64"]).max() <= 1e-5


@pytest.mark.gpu
def test_hip_adagrad_golden(cuda_device):
    from hades_amd import ops
    w = _d("ada_w0", cuda_device)
    s = torch.zeros_like(w)
    # rows addressed through a shuffled duplicate-free id list: the update is row-wise
    perm = torch.randperm(w.size(0), generator=torch.Generator().manual_seed(3)).to(cuda_device)
    for g in VEC["ada_g"]:
        gd = torch.from_numpy(g.copy()).to(cuda_device)[perm].contiguous()
        ops.adagrad_update_(perm, gd, None, None, w, s, None, 0.01, 1e-10)
    _adagrad_close(w.cpu().numpy(), s.cpu().numpy())


@pytest.mark.gpu
def test_hip_adam_golden(cuda_device):
    from hades_amd import ops
    w = _d("adam_w0", cuda_device)
    step = torch.zeros(w.size(0), dtype=torch.float32, device=cuda_device)
    m, v = torch.zeros_like(w), torch.zeros_like(w)
    uids = torch.arange(w.size(0), dtype=torch.int64, device=cuda_device)
    for g in VEC["adam_g"]:
        ops.adam_update_(uids, torch.from_numpy(g.copy()).to(cuda_device), None, (w, step, m, v),
                         None, 0.01, 0.9, 0.999, 1e-8)
    assert np.abs(m.cpu().numpy() - VEC["adam_m"]).max() <= 1e-9
    assert np.abs(v.cpu().numpy() - VEC["adam_v"]).max() <= 1e-12
    assert np.abs(w.cpu().numpy() - VEC["adam_w"]).max() <= 2e-4 * 0.01 * len(VEC["adam_g"])
    assert float(step[0]) == len(VEC["adam_g"])


@pytest.mark.gpu
def test_hip_accumulator_golden(cuda_device):
    from hades_amd import ops
    dim = VEC["acc_g0"].shape[1]
    acc = ops.ColdGradAccumulator(1024, dim, id_bound=1 << 30, device=cuda_device)
    for b in range(3):
        acc.accumulate(_d("acc_ids%d" % b, cuda_device), _d("acc_g%d" % b, cuda_device),
                       _d("acc_c%d" % b, cuda_device))
    ids, sums, cnts = acc.flush()
    assert _eq(ids.cpu().numpy(), VEC["acc_flush_ids"]) and _eq(cnts.cpu().numpy(), VEC["acc_flush_cnts"])
    # one add per slot per batch, in batch order: bit-exact
    assert _eq(sums.cpu().numpy(), VEC["acc_flush_sums"])
    ids2, _, _ = acc.flush()
    assert ids2.numel() == 0


@pytest.mark.gpu
@pytest.mark.parametrize("host_cold", [False, True])
def test_hip_split_schedule_golden(cuda_device, host_cold):
    from hades_amd import ops
    from hades_amd.sparse_optim import SparseAdagrad
    kb = int(VEC["ss_key_bits"][0])
    q = _d("ss_q", cuda_device)
    hs = ops.HotSet(_d("ss_hot", cuda_device))
    keys = torch.empty_like(q)
    loc, hot_pos, cold_pos, counts = ops.lookup_split(q, hs, sort_keys=keys, key_bits=kb)
    nh, nc = counts.tolist()
    assert _eq(loc.cpu().numpy(), VEC["ss_loc"]) and _eq(keys.cpu().numpy(), VEC["ss_keys"])
    assert _eq(hot_pos[:nh].cpu().numpy(), VEC["ss_hot_pos"]) and _eq(cold_pos[:nc].cpu().numpy(), VEC["ss_cold_pos"])
    first_pos = torch.empty(q.numel(), dtype=torch.int32, device=cuda_device)
    plan = ops.combine_plan_classed(keys, VEC["ss_grad"].shape[1], kb, first_pos=first_pos)
    g = _d("ss_grad", cuda_device)
    sums, cnts = ops.combine_apply_class(plan, g, 0, ops.COMBINE_EXACT)
    ops.combine_apply_class(plan, g, 1, ops.COMBINE_EXACT, out=(sums, cnts))
    U = int(plan.num_unique.item())
    assert _eq(plan.uids[:U].cpu().numpy(), VEC["ss_ukeys"]) and _eq(cnts[:U].cpu().numpy(), VEC["ss_ucnts"])
    assert _eq(sums[:U].cpu().numpy(), VEC["ss_usums"])
    assert _eq(plan.class_split.cpu().numpy(), VEC["ss_class_split"])
    assert _eq(first_pos[:U].cpu().numpy(), VEC["ss_first_pos"])
    # the whole step through the optimizer, cold table in HBM or in pinned host memory
    cold = torch.from_numpy(VEC["ss_cold"].copy())
    cold = cold.pin_memory() if host_cold else cold.to(cuda_device)
    opt = SparseAdagrad(cold, torch.from_numpy(VEC["ss_hot"].copy()), lr=0.01, eps=1e-10)
    opt.hot_w.copy_(_d("ss_hot_rows", cuda_device))
    assert ops.key_bits_for(opt.num_rows) == kb
    rows, state = opt.forward_keyed(q)
    want = np.stack([VEC["ss_hot_rows"][l] if l >= 0 else VEC["ss_cold"][x] for l, x in zip(VEC["ss_loc"], VEC["ss_q"])])
    assert _eq(rows.cpu().numpy(), want)
    opt.backward_keyed(state, g, mode=ops.COMBINE_EXACT)
    torch.cuda.synchronize()
    _keyed_close(opt.cold_w.cpu().numpy(), opt.cold_s.cpu().numpy(), opt.hot_w.cpu().numpy(), opt.hot_s.cpu().numpy())
