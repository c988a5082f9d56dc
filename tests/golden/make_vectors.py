"""Writes tests/golden/vectors.npz: small input/expected-output vectors for every function on the
embedding-cache path.

The expected outputs are made here with library routines and brute force only - numpy
searchsorted / nonzero / unique / add.at, Python dicts and loops, torch.optim.Adagrad / Adam on a
dense parameter - never with the oracle or the HIP library, so that both can be checked against
them.  The recipes are the ones the reference's own test scripts compare with:
`dst = src_data[src_index]` (test/test_cached_fetch.py:22), `dst_data[dst_index] = src`
(test/test_cached_set.py:22), `torch.nonzero(mask)` (test/test_split.py:30-37),
`torch.unique` + `index_add_` (python/EmbCache/sparse_optim.py:19-61) and the Adagrad / Adam row
updates (python/EmbCache/sparse_optim.py:590-685, 372-520).

    python tests/golden/make_vectors.py        # rewrites vectors.npz next to this file
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def lookup_case(rng):
    num_rows = 5000
    hot = np.sort(rng.choice(num_rows, 300, replace=False)).astype(np.int64)
    q = rng.integers(0, num_rows, 1000).astype(np.int64)
    q[:6] = [hot[0], hot[-1], max(hot[0] - 1, 0), min(hot[-1] + 1, num_rows - 1), 0, num_rows - 1]
    slot_of = {int(h): k for k, h in enumerate(hot)}            # brute force membership
    loc = np.array([slot_of.get(int(x), -1) for x in q], dtype=np.int64)
    return {"lookup_hot": hot, "lookup_q": q, "lookup_loc": loc}


def split_case(rng):
    num_rows = 3000
    table = rng.integers(0, 3, num_rows).astype(np.int64)      # 0 cold, 1 hot, 2 remote-cold
    ids = rng.integers(0, num_rows, 700).astype(np.int64)
    cls = table[ids]
    out = {"split_table": table, "split_ids": ids}
    for k in range(3):
        pos = np.nonzero(cls == k)[0].astype(np.int64)
        out["split_pos%d" % k] = pos
        out["split_ids%d" % k] = ids[pos]
    return out


def rows_case(rng):
    num_rows, dim = 2000, 8
    hot = np.sort(rng.choice(num_rows, 250, replace=False)).astype(np.int64)
    cold = rng.standard_normal((num_rows, dim)).astype(np.float32)
    hot_rows = rng.standard_normal((hot.size, dim)).astype(np.float32)   # differ from the cold copy
    q = rng.integers(0, num_rows, 600).astype(np.int64)
    # fetch: the row comes from the hot table when the id is hot, else from the cold table
    slot_of = {int(h): k for k, h in enumerate(hot)}
    dst = np.stack([hot_rows[slot_of[int(x)]] if int(x) in slot_of else cold[int(x)] for x in q])
    # set: distinct ids; hot ids land in the hot table only, the others in the cold table only
    sq = rng.choice(num_rows, 400, replace=False).astype(np.int64)
    src = rng.standard_normal((sq.size, dim)).astype(np.float32)
    cold_after, hot_after = cold.copy(), hot_rows.copy()
    for r, x in enumerate(sq):
        if int(x) in slot_of:
            hot_after[slot_of[int(x)]] = src[r]
        else:
            cold_after[int(x)] = src[r]
    return {"rows_hot": hot, "rows_cold": cold, "rows_hot_rows": hot_rows, "rows_q": q,
            "rows_fetch_dst": dst, "rows_set_q": sq, "rows_set_src": src,
            "rows_set_cold_after": cold_after, "rows_set_hot_after": hot_after}


def combine_case(rng):
    n, dim, n_ids = 2000, 16, 300
    pool = rng.choice(1 << 20, n_ids, replace=False).astype(np.int64)
    w = 1.0 / np.arange(1, n_ids + 1)
    idx = pool[rng.choice(n_ids, n, p=w / w.sum())]
    grad = (rng.standard_normal((n, dim)) * 1e-3).astype(np.float32)
    uids, inverse, cnts = np.unique(idx, return_inverse=True, return_counts=True)
    sums32 = np.zeros((uids.size, dim), dtype=np.float32)
    np.add.at(sums32, inverse, grad)                            # fp32, in order of appearance
    sums64 = np.zeros((uids.size, dim), dtype=np.float64)
    np.add.at(sums64, inverse, grad.astype(np.float64))
    return {"comb_idx": idx, "comb_grad": grad, "comb_uids": uids.astype(np.int64),
            "comb_inverse": inverse.astype(np.int64), "comb_cnts": cnts.astype(np.int64),
            "comb_sums_seq32": sums32, "comb_sums_f64": sums64}


def adagrad_case(rng):
    rows, dim, steps = 64, 16, 3
    w0 = (rng.standard_normal((rows, dim)) * 0.01).astype(np.float32)
    gs = (rng.standard_normal((steps, rows, dim)) * 1e-3).astype(np.float32)
    gs[1, 5] = 0.0                                              # a zero-gradient row
    p = torch.nn.Parameter(torch.from_numpy(w0.copy()))
    opt = torch.optim.Adagrad([p], lr=0.01, eps=1e-10)
    for t in range(steps):
        p.grad = torch.from_numpy(gs[t].copy())
        opt.step()
    return {"ada_w0": w0, "ada_g": gs, "ada_w": p.detach().numpy().copy(),
            "ada_s": opt.state[p]["sum"].numpy().copy()}


def adam_case(rng):
    rows, dim, steps = 48, 8, 4
    w0 = (rng.standard_normal((rows, dim)) * 0.01).astype(np.float32)
    gs = (rng.standard_normal((steps, rows, dim)) * 1e-3).astype(np.float32)
    p = torch.nn.Parameter(torch.from_numpy(w0.copy()))
    opt = torch.optim.Adam([p], lr=0.01, betas=(0.9, 0.999), eps=1e-8)
    for t in range(steps):
        p.grad = torch.from_numpy(gs[t].copy())
        opt.step()
    st = opt.state[p]
    return {"adam_w0": w0, "adam_g": gs, "adam_w": p.detach().numpy().copy(),
            "adam_m": st["exp_avg"].numpy().copy(), "adam_v": st["exp_avg_sq"].numpy().copy()}


def accumulator_case(rng):
    """Three duplicate-free batches into a dict, then everything out in id order."""
    dim, pool = 8, rng.choice(1 << 30, 500, replace=False).astype(np.int64)
    table = {}
    out = {}
    for b in range(3):
        ids = rng.choice(pool, 200, replace=False).astype(np.int64)
        g = (rng.standard_normal((ids.size, dim)) * 1e-3).astype(np.float32)
        c = rng.integers(1, 5, ids.size).astype(np.int64)
        out["acc_ids%d" % b], out["acc_g%d" % b], out["acc_c%d" % b] = ids, g, c
        for r, x in enumerate(ids):
            s, k = table.get(int(x), (np.zeros(dim, np.float32), 0))
            table[int(x)] = ((s + g[r]).astype(np.float32), k + int(c[r]))
    keys = sorted(table)
    out["acc_flush_ids"] = np.array(keys, dtype=np.int64)
    out["acc_flush_sums"] = np.stack([table[k][0] for k in keys]).astype(np.float32)
    out["acc_flush_cnts"] = np.array([table[k][1] for k in keys], dtype=np.int64)
    return out


def split_schedule_case(rng):
    """One training step done class by class (split first: python/EmbCache/dist_emb.py:174-211),
    all by loops and dicts: slots, the two position lists, the class-ordered sort keys, the
    distinct keys with their sequential float32 sums and counts, the class border, and the tables
    after one Adagrad step (torch.optim.Adagrad on the gathered rows of each class)."""
    num_rows, dim, key_bits = 1500, 8, 11
    hot = np.sort(rng.choice(num_rows, 200, replace=False)).astype(np.int64)
    w = 1.0 / np.arange(1, num_rows + 1)
    q = rng.permutation(num_rows)[rng.choice(num_rows, 900, p=w / w.sum())].astype(np.int64)
    grad = (rng.standard_normal((q.size, dim)) * 1e-3).astype(np.float32)
    cold = (rng.standard_normal((num_rows, dim)) * 0.01).astype(np.float32)
    hot_rows = (rng.standard_normal((hot.size, dim)) * 0.01).astype(np.float32)
    slot_of = {int(h): k for k, h in enumerate(hot)}
    loc = np.array([slot_of.get(int(x), -1) for x in q], dtype=np.int64)
    hot_pos = np.array([p for p, x in enumerate(q) if int(x) in slot_of], dtype=np.int64)
    cold_pos = np.array([p for p, x in enumerate(q) if int(x) not in slot_of], dtype=np.int64)
    keys = np.array([(1 << key_bits) | slot_of[int(x)] if int(x) in slot_of else int(x) for x in q],
                    dtype=np.int64)
    sums, cnts, first = {}, {}, {}
    for p, k in enumerate(keys):                                  # occurrence order, float32
        k = int(k)
        sums[k] = (sums.get(k, np.zeros(dim, np.float32)) + grad[p]).astype(np.float32)
        cnts[k] = cnts.get(k, 0) + 1
        first.setdefault(k, p)
    ukeys = np.array(sorted(sums), dtype=np.int64)
    usums = np.stack([sums[int(k)] for k in ukeys]).astype(np.float32)
    ucnts = np.array([cnts[int(k)] for k in ukeys], dtype=np.int64)
    ufirst = np.array([first[int(k)] for k in ukeys], dtype=np.int32)
    split_run = int(sum(1 for k in ukeys if k < (1 << key_bits)))
    cold_after, hot_after = cold.copy(), hot_rows.copy()
    cold_state, hot_state = np.zeros_like(cold), np.zeros_like(hot_rows)
    for table, state, rows, g in ((cold_after, cold_state, ukeys[:split_run], usums[:split_run]),
                                  (hot_after, hot_state, ukeys[split_run:] - (1 << key_bits), usums[split_run:])):
        prm = torch.nn.Parameter(torch.from_numpy(table[rows].copy()))
        opt = torch.optim.Adagrad([prm], lr=0.01, eps=1e-10)
        prm.grad = torch.from_numpy(g.copy())
        opt.step()
        table[rows] = prm.detach().numpy()
        state[rows] = opt.state[prm]["sum"].numpy()
    return {"ss_hot": hot, "ss_q": q, "ss_grad": grad, "ss_cold": cold, "ss_hot_rows": hot_rows,
            "ss_key_bits": np.array([key_bits], np.int64), "ss_loc": loc, "ss_hot_pos": hot_pos,
            "ss_cold_pos": cold_pos, "ss_keys": keys, "ss_ukeys": ukeys, "ss_usums": usums,
            "ss_ucnts": ucnts, "ss_first_pos": ufirst,
            "ss_class_split": np.array([cold_pos.size, split_run], np.int64),
            "ss_cold_after": cold_after, "ss_hot_after": hot_after, "ss_cold_state": cold_state,
            "ss_hot_state": hot_state}


def main():
    rng = np.random.default_rng(20240611)
    torch.manual_seed(0)
    vec = {}
    for case in (lookup_case, split_case, rows_case, combine_case, adagrad_case, adam_case,
                 accumulator_case, split_schedule_case):      # new cases go last: the earlier
        # arrays depend on the generator's position and must not change
        vec.update(case(rng))
    path = os.path.join(HERE, "vectors.npz")
    np.savez_compressed(path, **vec)
    print("wrote %s (%d arrays, %d bytes)" % (path, len(vec), os.path.getsize(path)))


if __name__ == "__main__":
    main()
