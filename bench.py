"""Benchmark of the embedding-cache hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]      the headline workload (cfg3) + cfg2 nested
    python bench.py --workload cfg2|cfg3|cfg5 [--mode fast|exact] [--schedule serial|keyed|pipelined|split|overlap|graph]
                    [--no-reuse-rows] [--optimizer adagrad|adam]
    python bench.py --workload cfg4          cold-gradient accumulator with delayed write-back
    python bench.py --workload cfg4 --flush-rule staleness    the cache server's own per-row rule
    python bench.py --workload neighbours    pre-exchange bucketing, index cache, cold-data cache
    python bench.py --workload random-rows   what distinct random 512-byte rows of a 2 GB table cost
    python bench.py --workload host-link     what the host link gives kernels: rows, grid width, burst, direction

One step = lookup + cached_fetch of the query rows, combine of the per-query gradients, and the
sparse Adagrad update of every distinct row, on one batch of synthetic Zipf ids that is already
resident in HBM.  The headline workload keeps 10 % of a 111 M x 128 table in HBM and the rest in
pinned host memory; its step runs on the keyed schedule: one lookup + stable hot/cold partition per
query batch, then the hot rows through kernels that only touch HBM and the cold rows through narrow
kernels that only touch the host table, on two streams; the combine sorts class-ordered keys, so
the cold class is summed first and its update crosses the host link while the hot class is still
being summed and updated.  Prints ONE JSON line: whole-step throughput in query rows/s
(mean, median, p10/p90 over the timed steps), the HBM roofline of every row kernel (algorithmic
bytes / HIP-event time of its launches inside the timed region), the host-link roofline of the
cold-row kernels against the nominal 64 GB/s and against pinned hipMemcpyAsync rates measured in
the same run, and the same step timed on the host cores with the CPU oracle.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
PCIE_PEAK_GBS = 64.0


def measured_traffic(workload, mode):
    """HBM bytes per launch from the committed rocprofv3 counter summary of this workload
    (profiles/<workload>_step_hbm_traffic.txt, lines `TRAFFIC kernel=<key> bytes=<n>`), or {} if
    there is none: hardware counters cannot be read from inside this script."""
    path = os.path.join(ROOT, "profiles", "%s_step_hbm_traffic.txt" % workload)
    out = {}
    if mode != "fast" or not os.path.exists(path):
        return out
    with open(path) as f:
        for line in f:
            m = re.match(r"\s*TRAFFIC\s+kernel=(\S+)\s+bytes=([0-9.eE+]+)", line)
            if m:
                out[m.group(1)] = float(m.group(2))
    return out


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="cfg3", choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg5", "neighbours", "random-rows", "host-link"])
    ap.add_argument("--mode", default="fast", choices=["fast", "exact"])
    ap.add_argument("--optimizer", default="adagrad", choices=["adagrad", "adam"],
                    help="row update of the step: sparse Adagrad (the configurations' optimizer) or "
                         "the reference's SparseAdam (cfg2 / cfg3 / cfg5 steps only)")
    ap.add_argument("--schedule", default=None, choices=["serial", "keyed", "pipelined", "split", "overlap", "graph"],
                    help="serial: every kernel of the step on one stream, hot and cold rows in the "
                         "same kernels (default when the whole table is in HBM); keyed: one lookup + "
                         "hot/cold partition per batch, hot rows on one stream, cold rows on "
                         "another, combine over class-ordered keys so that the cold update starts "
                         "first (default when the cold table is in host memory); split: the same "
                         "two streams with a plain combine and a second lookup of the distinct "
                         "ids; overlap: serial with the sort of "
                         "the ids on a side stream next to the fetch; graph: serial, every step the "
                         "replay of a HIP graph captured once per batch")
    ap.add_argument("--no-reuse-rows", dest="reuse_rows", action="store_false",
                    help="keyed / pipelined schedules: make the cold update read the old weight rows "
                         "from the host table again.  By default it takes them from the rows the "
                         "step's own fetch brought in whenever the optimizer can tell that nothing "
                         "has written the table in between (backward_keyed's guarded default)")
    ap.add_argument("--cold-state", default="hbm", choices=["hbm", "host"],
                    help="cfg3 with Adagrad: where the cold optimizer state lives.  hbm (default): "
                         "the full 111 M-row table, cold weights in pinned host memory, cold state "
                         "in HBM.  host: the contract layout - weights and state both in pinned host "
                         "memory, side by side in one [N, 2, D] table - on a table cut to half the "
                         "rows, which is what one page-locked allocation of this box holds")
    ap.add_argument("--average", default=None, choices=["sum", "mean", "one_plus"],
                    help="what the update applies for an id that occurs several times in a batch: the "
                         "sum of its gradient rows (the configurations' combine; default for Adagrad), "
                         "or their mean as the reference's update does (unique_grads; default for "
                         "--optimizer adam), or the sum over one plus the occurrences")
    ap.add_argument("--sort", default=None, choices=["one-sweep", "three-kernels"],
                    help="form of the radix sort under the combine (default: the library's)")
    ap.add_argument("--allow-fallback", action="store_true",
                    help="if the host refuses cfg3's page-locked table, measure cfg2 instead and say "
                         "so in config.fallback (without this flag such a run exits non-zero)")
    ap.add_argument("--flush-rule", default="every8", choices=["every8", "staleness"],
                    help="cfg4 only: write the accumulated cold gradients back every 8 steps (hash "
                         "accumulator), or per row by the cache server's staleness rule (cold-data "
                         "cache)")
    ap.add_argument("--batches", type=int, default=4, help="distinct pre-generated id batches")
    ap.add_argument("--event-every", type=int, default=4,
                    help="bracket the row kernels with HIP events in every n-th timed step")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true",
                    help="headline run only: skip the nested cfg2 measurement")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run three plain 256 MiB device copies before the timed region "
                         "(a known-size reference for hardware byte counters)")
    return ap.parse_args()


def log(msg):
    """Progress on stderr (stdout carries only the JSON line)."""
    print("[bench %6.1fs] %s" % (time.perf_counter() - _T0, msg), file=sys.stderr, flush=True)


_T0 = time.perf_counter()


def pct(xs, p):
    """p-th percentile (linear interpolation) of a list."""
    xs = sorted(xs)
    if not xs:
        return float("nan")
    k = (len(xs) - 1) * p / 100.0
    lo = int(k)
    hi = min(lo + 1, len(xs) - 1)
    return xs[lo] + (xs[hi] - xs[lo]) * (k - lo)


class Workload:
    """Tables, hot set and pre-generated batches of one configuration, resident on the device
    (cold table in pinned host memory for cfg3)."""

    def __init__(self, name, nbatches, device, optimizer="adagrad", state_on_host=False):
        import torch
        from hades_amd import synth
        from hades_amd.sparse_optim import SparseAdagrad, SparseAdam
        self.optimizer = optimizer
        cfg = synth.CONFIGS[name]
        self.name, self.cfg = name, cfg
        N, D, H = cfg["num_rows"], cfg["dim"], cfg["num_hot"]
        # state_on_host (cfg3, Adagrad): the contract layout - cold weights AND cold optimizer
        # state in pinned host memory - on a table cut to half the rows, so that one page-locked
        # allocation of the size the box grants holds both, side by side: [N/2, 2, D], the weight
        # row and the state row of an id in one 1 KB stretch.  Batch, skew and hot fraction stay.
        self.state_on_host = bool(state_on_host) and name == "cfg3" and optimizer == "adagrad"
        if self.state_on_host:
            N, H = N // 2, H // 2
        self.N, self.D, self.H = N, D, H
        self.trainers = cfg.get("trainers", 1)
        self.n = cfg["batch"] * self.trainers
        self.host_cold = name == "cfg3"
        seed = 1234 + int(name[3:])
        log("allocating the %d x %d table (%.1f GB, %s)" %
            (N, D, N * D * 4 * (2 if self.state_on_host else 1) / 1e9,
             "pinned host, weight and state rows interleaved" if self.state_on_host
             else "pinned host" if self.host_cold else "HBM"))
        both = None
        if self.state_on_host:
            both = torch.empty((N, 2, D), dtype=torch.float32, pin_memory=True)
            table = both[:, 0]
        elif self.host_cold:
            table = torch.empty((N, D), dtype=torch.float32, pin_memory=True)
        else:
            table = torch.empty((N, D), dtype=torch.float32, device=device)
        log("filling it")
        if both is not None:
            synth.fill_interleaved_(both, 0.01, seed, progress=log)
        else:
            synth.fill_normal_(table, 0.01, seed, progress=log if N > 50_000_000 else None)
        hot_ids = synth.hot_ids(N, H, device) if H else torch.empty(0, dtype=torch.int64, device=device)
        log("hot copies and optimizer state")
        # cfg3: the cold weights are the pinned host table; the cold Adagrad state stays in HBM.
        # The benchmark box refuses a page-locked allocation that would hold weights and state
        # together (113.7 GB in one piece: hipHostMalloc says out of memory; 56.8 GB is granted),
        # and 288 GB of HBM have the room.
        if optimizer == "adam":      # its cold step / mem / power tables stay in HBM likewise
            self.opt = SparseAdam(table, hot_ids, lr=0.01, betas=(0.9, 0.999), eps=1e-8, device=device,
                                  state_on_device=self.host_cold)
        elif both is not None:
            self.opt = SparseAdagrad(table, hot_ids, lr=0.01, eps=1e-10, device=device,
                                     cold_state=both[:, 1])
        else:
            self.opt = SparseAdagrad(table, hot_ids, lr=0.01, eps=1e-10, device=device,
                                     state_on_device=self.host_cold)
        log("sampling %d batches of %d ids" % (nbatches, self.n))
        sampler = synth.ZipfSampler(N, cfg["zipf_s"], device)
        self.ids, self.grads = [], []
        for b in range(nbatches):
            parts = [synth.make_ids(sampler, N, cfg["batch"], seed * 1000 + b * 16 + t)
                     for t in range(self.trainers)]
            self.ids.append(torch.cat(parts).contiguous())
            self.grads.append(synth.make_grads(self.n, D, seed * 2000 + b, device))
        del sampler
        self.rows_out = torch.empty((self.n, D), dtype=torch.float32, device=device)
        self.comb_out = (torch.empty(self.n, dtype=torch.int64, device=device),
                         torch.empty((self.n, D), dtype=torch.float32, device=device),
                         torch.empty(self.n, dtype=torch.int64, device=device),
                         torch.empty(1, dtype=torch.int64, device=device))
        log("workload ready")

    def describe(self):
        return ("%s: %d x %d fp32 table (%s), hot %d rows in HBM, %d ids/step zipf s=%.2f%s" %
                (self.name, self.N, self.D,
                 "cold weights and cold Adagrad state both in pinned host memory, read and written "
                 "zero-copy, the two rows of an id side by side in one [N, 2, D] table; deviation: "
                 "the table is cut to half of cfg3's rows so that the one page-locked allocation the "
                 "box grants holds both" if self.state_on_host else
                 "cold weights in pinned host memory read and written zero-copy; deviation: cold "
                 "optimizer state in HBM, the box refuses the 113.7 GB page-locked allocation that "
                 "would hold weights and state" if self.host_cold
                 else "all in HBM", self.H, self.n, self.cfg["zipf_s"],
                 ", %d trainer batches concatenated" % self.trainers if self.trainers > 1 else ""))


class WorkloadSetupError(RuntimeError):
    """The tables of a workload could not be allocated on this host / GPU."""


def link_probe(dev, nbytes=128 << 20, reps=4):
    """Pinned hipMemcpyAsync rates of this box, GB/s: host to device, device to host, and each
    direction while the other runs on a second stream."""
    import torch
    h1 = torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)
    h2 = torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)
    d1 = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    d2 = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    from hades_amd.sparse_optim import side_stream     # no further streams: see side_stream
    s1, s2 = side_stream(dev, 0), side_stream(dev, 1)

    def h2d():
        with torch.cuda.stream(s1):
            d1.copy_(h1, non_blocking=True)

    def d2h():
        with torch.cuda.stream(s2):
            h2.copy_(d2, non_blocking=True)

    def rate(fns):
        for f in fns:
            f()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            for f in fns:
                f()
        torch.cuda.synchronize()
        return nbytes * reps / (time.perf_counter() - t0) / 1e9

    out = {"h2d_GB/s": round(rate([h2d]), 2), "d2h_GB/s": round(rate([d2h]), 2),
           "both_ways_each_GB/s": round(rate([h2d, d2h]), 2),
           "note": "pinned hipMemcpyAsync of %d MiB, %d repetitions" % (nbytes >> 20, reps)}
    del h1, h2, d1, d2
    return out


def link_kernel_probe(wl, reps=3):
    """What the host link gives kernels on this box for the workload's own cold rows (batch 0):
    the listed gather alone (host -> HBM), the listed scatter alone (HBM -> host; it writes back
    the rows just read, so the table does not change), and both at once on two streams."""
    import torch
    from hades_amd import ops
    opt = wl.opt
    q = wl.ids[0]
    loc, hot_pos, cold_pos, counts = ops.lookup_split(q, opt.hot_set)
    n_cold = int(counts[1].item())
    cnt = counts[1:2]
    rows = wl.rows_out
    ops.fetch_listed(opt.cold_w, q, cold_pos, cnt, rows)
    src = rows.clone()
    from hades_amd.sparse_optim import side_stream
    s1, s2 = side_stream(opt.device, 0), side_stream(opt.device, 1)
    mb = n_cold * wl.D * 4 / 1e6

    def gather():
        with torch.cuda.stream(s1):
            ops.fetch_listed(opt.cold_w, q, cold_pos, cnt, rows)

    def scatter():
        with torch.cuda.stream(s2):
            ops.set_listed(src, opt.cold_w, q, cold_pos, cnt)

    def rate(fns):
        best = 0.0
        for _ in range(reps + 1):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for f in fns:
                f()
            torch.cuda.synchronize()
            best = max(best, mb / ((time.perf_counter() - t0) * 1e3))
        return round(best, 2)

    out = {"rows": n_cold, "gather_GB/s": rate([gather]), "scatter_GB/s": rate([scatter]),
           "both_ways_each_GB/s": rate([gather, scatter]),
           "note": "listed gather / scatter kernels over the cold rows of batch 0, wall clock "
                   "around one call (launch latency included), best of %d" % (reps + 1)}
    del src
    return out


def parity_gate(wl, step_fn, rows=20_000, average=None, rows_are_sums=True):
    """One untimed step in the deterministic-order mode on the first `rows` ids of batch 0,
    through the same schedule as the timed steps, checked against torch's own device operators:
    slots and fetched rows bit-exact, distinct ids and counts exact, summed gradients and the
    updated weight / state rows within 1e-5 relative per row.  Raises on a mismatch."""
    import torch
    from hades_amd import ops
    opt = wl.opt
    m = min(rows, wl.n)
    q = wl.ids[0][:m].contiguous()
    g = wl.grads[0][:m].contiguous()
    hot = opt.hot_ids

    def table_rows(cold, hot_t, ids):
        """rows of (cold, hot_t) named by ids, gathered with torch indexing only"""
        pos = torch.searchsorted(hot, ids, right=True)
        hit = (pos > 0) & (hot[(pos - 1).clamp_(min=0)] == ids) if hot.numel() else torch.zeros_like(ids, dtype=torch.bool)
        loc = torch.where(hit, pos - 1, torch.full_like(pos, -1))
        out = torch.empty((ids.numel(), wl.D), dtype=torch.float32, device=ids.device)
        if hot.numel():
            out[hit] = hot_t[loc[hit]]
        miss = ~hit
        if cold.is_cuda:
            out[miss] = cold[ids[miss]]
        else:
            out[miss] = cold[ids[miss].cpu()].to(ids.device)
        return out, loc

    want_rows, want_loc = table_rows(opt.cold_w, opt.hot_w, q)
    got_loc = ops.lookup(q, opt.hot_set)
    assert torch.equal(got_loc, want_loc), "parity gate: lookup slots differ"
    uniq, inv, cnt = torch.unique(q, sorted=True, return_inverse=True, return_counts=True)
    sums64 = torch.zeros((uniq.numel(), wl.D), dtype=torch.float64, device=q.device)
    sums64.index_add_(0, inv, g.double())
    w0, _ = table_rows(opt.cold_w, opt.hot_w, uniq)
    adam = wl.optimizer == "adam"
    if adam:
        m0, loc_u = table_rows(opt.cold_m, opt.hot_m, uniq)
        v0, _ = table_rows(opt.cold_v, opt.hot_v, uniq)

        def steps_of():
            hit = loc_u >= 0
            st = opt.cold_step[uniq].clone()
            if hot.numel():
                st[hit] = opt.hot_step[loc_u[hit]]
            return st
        st0 = steps_of()
    else:
        s0, _ = table_rows(opt.cold_s, opt.hot_s, uniq)

    rows_out, (uids, sums, cnts, nu) = step_fn(q, g, ops.COMBINE_EXACT)
    torch.cuda.synchronize()
    assert torch.equal(rows_out[:m], want_rows), "parity gate: fetched rows differ"
    u = int(nu.item())
    assert u == uniq.numel() and torch.equal(uids[:u], uniq), "parity gate: distinct ids differ"
    assert torch.equal(cnts[:u], cnt), "parity gate: counts differ"

    def close(a, b, what):
        err = (a.double() - b.double()).abs().amax(dim=1)
        scale = b.double().abs().amax(dim=1).clamp_(min=1e-30)
        worst = float((err / scale).max())
        assert worst <= 1e-5, "parity gate: %s off by %.3g relative" % (what, worst)
        return worst

    # the keyed schedule returns the sums and divides inside its update kernels; the other
    # schedules divide the combined rows in place before the update
    div = (cnt + (1 if average == "one_plus" else 0)).to(torch.float32).unsqueeze(1) if average else None
    if average and not rows_are_sums:
        e_sum = close(sums[:u], sums64 / div.double(), "averaged gradients")
        gs = sums[:u]
    else:
        e_sum = close(sums[:u], sums64, "summed gradients")
        gs = sums[:u] / div if average else sums[:u]
    w_got, _ = table_rows(opt.cold_w, opt.hot_w, uniq)
    if adam:
        # the reference's float32 arithmetic (python/EmbCache/sparse_optim.py:632-657,681) in torch
        b1, b2 = opt.betas
        st1 = st0 + 1
        m1 = b1 * m0 + (1.0 - b1) * gs
        v1 = b2 * v0 + (1.0 - b2) * (gs * gs)
        c1 = (1.0 - torch.pow(torch.tensor(b1, device=q.device), st1)).unsqueeze(1)
        c2 = (1.0 - torch.pow(torch.tensor(b2, device=q.device), st1)).unsqueeze(1)
        w1 = w0 - 0.01 * (m1 / c1) / (torch.sqrt(v1 / c2) + opt.eps)
        m_got, _ = table_rows(opt.cold_m, opt.hot_m, uniq)
        v_got, _ = table_rows(opt.cold_v, opt.hot_v, uniq)
        assert torch.equal(steps_of(), st1), "parity gate: Adam step counters differ"
        errs = {"sums": e_sum, "weights": close(w_got, w1, "updated weights"),
                "mem": close(m_got, m1, "updated Adam mem"), "power": close(v_got, v1, "updated Adam power")}
        form = "SparseAdam closed form in float32, first step of every row"
    else:
        s1 = s0 + gs * gs
        w1 = w0 - (0.01 * gs) / (s1.sqrt() + 1e-10)
        s_got, _ = table_rows(opt.cold_s, opt.hot_s, uniq)
        errs = {"sums": e_sum, "weights": close(w_got, w1, "updated weights"),
                "state": close(s_got, s1, "updated Adagrad state")}
        form = "Adagrad closed form"
    return {"rows": m, "distinct": u, "mode": "exact",
            "bit_exact": ["lookup slots", "fetched rows", "distinct ids", "counts"] +
                         (["Adam step counters"] if adam else []),
            "max_rel_err": errs, "tolerance": 1e-5,
            "against": "torch device ops (searchsorted, indexing, unique + float64 index_add_, %s)" % form}


def run_gpu(args, workload, schedule, with_gate=True, with_link=True, reuse_rows=True,
            state_on_host=False):
    import torch
    from hades_amd import ops
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    try:
        wl = Workload(workload, args.batches, dev, args.optimizer, state_on_host=state_on_host)
    except (RuntimeError, MemoryError) as err:
        msg = str(err).splitlines()[0][:300] if str(err) else type(err).__name__
        if "memory" in msg.lower():
            raise WorkloadSetupError(msg) from err
        raise
    if args.sort is not None:
        ops.sort_config(one_sweep=args.sort == "one-sweep")
    opt = wl.opt
    mode = ops.COMBINE_FAST if args.mode == "fast" else ops.COMBINE_EXACT
    nb = len(wl.ids)
    n, D, N = wl.n, wl.D, wl.N
    K = args.steps
    if schedule is None:
        schedule = "keyed" if wl.host_cold else "serial"
    split = schedule == "split"
    pipelined = schedule == "pipelined"
    keyed = schedule == "keyed" or pipelined     # pipelined: the keyed kernels, two batches in flight
    overlap = schedule == "overlap"

    def new_events(count):
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(count)]
        for e in evs:
            e.record()          # torch creates the HIP event on first use
        return evs

    uids_o, sums_o, cnts_o, nu_o = wl.comb_out
    average = args.average if args.average is not None else ("mean" if args.optimizer == "adam" else None)
    average = None if average == "sum" else average
    reused = {"yes": 0, "no": 0}    # backward halves that took / did not take the forward rows

    def run_step(q, g, cmode, events=None, timing=None):
        """fetch -> combine -> update of one batch.

        serial: one stream; hot and cold rows share the fetch kernel and the update kernel.
        overlap: serial, but the id-only half of the combine (sort + run boundaries) is issued on
        a side stream before the fetch, as a trainer that knows the ids at forward time would do.
        split: lookup + hot/cold partition; the hot gather on the main stream and the cold gather
        on the cold stream; the id-only half of the combine runs on the main stream meanwhile
        (it needs the ids only); join: the fetched rows are complete, which is where a trainer's
        forward and backward would sit; segmented sum of the gradients; lookup + partition of the
        distinct ids; hot update on the main stream and cold update on the cold stream; join."""
        sizes = q.numel()
        rows = wl.rows_out[:sizes]
        out_ids = (uids_o[:sizes], nu_o)
        out_sum = (sums_o[:sizes], cnts_o[:sizes])
        if events: events[0].record()
        if keyed:
            # forward: lookup + partition + both gathers + sort of the class-ordered keys; the
            # join inside it is where a trainer's forward and backward would sit.  backward: cold
            # sums, cold update on the cold stream, hot sums and hot update beside it, join.
            _, state = opt.forward_keyed(q, out=rows, timing=timing)
            if events: events[1].record()
            if events: events[2].record()
            res = opt.backward_keyed(state, g, cmode, timing=timing,
                                     fetched_rows="auto" if reuse_rows else None, average=average)
            reused["yes" if state[0].reused_rows else "no"] += 1
        elif split:
            opt.fetch_split(q, out=rows, join=False, timing=timing)
            plan = ops.combine_plan(q, D, id_bound=N, workspace=opt._ws, out=out_ids)
            opt.join()
            if events: events[1].record()
            res = ops.combine_apply(plan, g, cmode, out=out_sum)
            if events: events[2].record()
            opt.update_split(res[0], res[1], res[3], join=True, timing=timing, cnts=res[2],
                             average=average)
        else:
            if overlap:
                plan = opt.prepare(q, out=out_ids)
            ops.cached_fetch(opt.cold_w, opt.hot_w, q, opt.hot_set, out=rows)
            if events: events[1].record()
            if overlap:
                torch.cuda.current_stream().wait_event(plan.ready)
            else:
                plan = ops.combine_plan(q, D, id_bound=N, workspace=opt._ws, out=out_ids)
            res = ops.combine_apply(plan, g, cmode, out=out_sum)
            if events: events[2].record()
            opt.update(res[0], res[1], res[3], cnts=res[2], average=average)
        if events: events[3].record()
        return rows, res

    # pipelined schedule: step i = the forward half of batch i+1 started on side streams
    # (prefetch_keyed), the backward half of batch i, then the completion of batch i+1's rows
    # (hot gather behind the hot update, refresh of the cold rows that update wrote).  `pipe`
    # carries batch i's rows and plan from step to step; a step whose batch is not the one in
    # flight runs that batch's forward half first (only ever extra work).
    pipe = {"i": None}
    row_bufs = [wl.rows_out, torch.empty_like(wl.rows_out)] if pipelined else None

    def prime(i):
        rows, st = opt.forward_keyed(wl.ids[i % nb], out=row_bufs[i % 2], slot=i % 2)
        pipe.update(i=i, rows=rows, state=st)

    def pipe_step(i, cmode, events=None, timing=None):
        if pipe["i"] != i:
            prime(i)
        rows, st = pipe["rows"], pipe["state"]
        if events: events[0].record()
        nxt = opt.prefetch_keyed(wl.ids[(i + 1) % nb], slot=(i + 1) % 2, out=row_bufs[(i + 1) % 2],
                                 timing=timing)
        if events: events[1].record()
        if events: events[2].record()
        res = opt.backward_keyed(st, wl.grads[i % nb], cmode, timing=timing,
                                 fetched_rows="auto" if reuse_rows else None, join=False,
                                 average=average)
        reused["yes" if st[0].reused_rows else "no"] += 1
        rows2, st2 = opt.finish_prefetch(nxt, after=st, timing=timing)
        if events: events[3].record()
        pipe.update(i=i + 1, rows=rows2, state=st2)
        return rows, res

    def step(i, events=None, timing=None):
        if pipelined:
            pipe_step(i, mode, events, timing)
        else:
            run_step(wl.ids[i % nb], wl.grads[i % nb], mode, events, timing)

    def gate_step(q, g, m):
        """one step for the parity gate: rows and the distinct rows in id order"""
        if pipelined:
            # batch (q, g) through the pipelined calls, with the same ids prefetched as the next
            # batch: every cold row of that next batch is written by this batch's update, so its
            # rows are right only if the refresh works - checked against the one-kernel fetch
            rows, st = opt.forward_keyed(q, out=row_bufs[0][:q.numel()], slot=0)
            rows = rows.clone()
            nxt = opt.prefetch_keyed(q, slot=1, out=row_bufs[1][:q.numel()])
            res = opt.backward_keyed(st, g, m, fetched_rows="auto" if reuse_rows else None, join=False,
                                     average=average)
            rows2, _ = opt.finish_prefetch(nxt, after=st)
            torch.cuda.synchronize()
            want2 = ops.cached_fetch(opt.cold_w, opt.hot_w, q, opt.hot_set)
            assert torch.equal(rows2, want2), "parity gate: rows prefetched across an update differ"
            pipe["i"] = None
        else:
            rows, res = run_step(q, g, m)
        if keyed:
            ukeys, sums, cnts, nu, _ = res
            ids = opt.distinct_ids_of(ukeys, nu)
            order = torch.argsort(ids)
            u = ids.numel()
            return rows, (ids[order], sums[:u][order], cnts[:u][order], nu)
        return rows, res

    gate = None
    if with_gate:
        gate = parity_gate(wl, gate_step, average=average, rows_are_sums=not split)
        log("parity gate passed: %s" % json.dumps(gate["max_rel_err"]))
    link = None
    if with_link and wl.host_cold:
        # the probes need page-locked buffers of their own next to the 56.8 GB table: a host that
        # has none left loses the probes, not the measurement
        try:
            link = link_probe(dev)
            link["kernels"] = link_kernel_probe(wl)
            log("host link: %s" % json.dumps(link))
        except (RuntimeError, MemoryError) as err:
            link = None
            log("host-link probes skipped: %s" % (str(err).splitlines()[0][:200] if str(err) else type(err).__name__))
            torch.cuda.empty_cache()

    for i in range(args.warmup):
        step(i)
    if args.copy_probe:
        a = torch.empty(64 << 20, dtype=torch.float32, device=dev).normal_()
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        del a, b
    torch.cuda.synchronize()

    # ---- the row kernels and how each is bracketed ----
    # split: the four listed kernels by event pairs recorded from Python on their own stream, the
    # segmented sum by the library's hook; serial: all three by the hook, one kernel per sampled
    # step in rotation (the hook brackets one kernel at a time).
    every = max(1, args.event_every)
    sampled = [i for i in range(K) if i % every == 0]
    seg_name = "seg_chunk_kernel" if args.mode == "fast" else "seg_exact_kernel + seg_exact_long_kernel"
    if split or keyed:
        oname = args.optimizer
        upd = "hades_%s_update_class" % oname if keyed else "hades_%s_update_listed" % oname
        knames = {"hot_fetch": "row_move_listed_kernel<gather> over the hot class (hades_fetch_listed)",
                  "cold_fetch": "row_move_listed_kernel<gather> over the cold class (hades_fetch_listed)",
                  "seg_sum": seg_name + (" over the hot class (hades_combine_apply_class)" if keyed
                                         else " (hades_combine_apply)"),
                  "hot_update": "%s_listed_kernel over the hot class (%s)" % (oname, upd),
                  "cold_update": "%s_listed_kernel over the cold class (%s)" % (oname, upd)}
        if pipelined:
            knames["cold_refresh"] = ("row_move_listed_kernel<gather, filter>: the next batch's cold rows "
                                      "that this batch's update wrote, read again (hades_fetch_listed_in_set)")
        hook_of = {"seg_sum": ops.KERNEL_SEG_SUM}
    else:
        knames = {"fetch": "row_move_kernel<AddrFetchSorted> (hades_cached_fetch)",
                  "seg_sum": seg_name + " (hades_combine_apply)",
                  "update": "%s_kernel (hades_%s_update)" % (args.optimizer, args.optimizer)}
        hook_of = {"fetch": ops.KERNEL_CACHED_FETCH, "seg_sum": ops.KERNEL_SEG_SUM,
                   "update": ops.KERNEL_ADAM if args.optimizer == "adam" else ops.KERNEL_ADAGRAD}
    kev = {i: {k: new_events(2) for k in knames} for i in sampled}
    step_ev = new_events(K + 1)
    phase_ev = [new_events(4) for _ in range(K)]
    torch.cuda.synchronize()
    hooks = sorted(hook_of)
    armed = {}

    kernel_ms = {k: [] for k in knames}
    if schedule == "graph":
        # one captured graph per pre-generated batch (the library allocates nothing and clears
        # memory with kernels only, so a step captures as it is); launches inside a replay cannot
        # be bracketed, so the kernels are timed on eager steps before the timed region
        for j, i in enumerate(sampled):
            hk = hooks[j % len(hooks)]
            ops.profile_kernel(hook_of[hk], kev[i][hk][0], kev[i][hk][1])
            step(i)
            armed[i] = [hk]
        ops.profile_kernel(0)
        graphs = []
        from hades_amd.sparse_optim import side_stream
        side = side_stream(dev, 0)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for b in range(nb):
                gr = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gr, stream=side):
                    step(b)
                graphs.append(gr)
        torch.cuda.current_stream().wait_stream(side)
        for b in range(nb):
            graphs[b].replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        step_ev[0].record()
        for i in range(K):
            graphs[i % nb].replay()
            step_ev[i + 1].record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    else:
        # Timed region: exactly K steps.  One event record per step marks the step boundary
        # (3-4 us of GPU time each, inside the measured time); the kernel brackets are taken in
        # every `event_every`-th step only.
        if pipelined:       # batch 0's forward half: the pipeline is full when the clock starts
            prime(0)
            torch.cuda.synchronize()
        t0 = time.perf_counter()
        step_ev[0].record()
        for j_i, i in enumerate(range(K)):
            tim = None
            if i % every == 0:
                j = i // every
                if split or keyed:
                    tim = {k: kev[i][k] for k in knames if k not in hook_of}
                    hk = "seg_sum"
                    armed[i] = list(knames)
                else:
                    hk = hooks[j % len(hooks)]
                    armed[i] = [hk]
                ops.profile_kernel(hook_of[hk], kev[i][hk][0], kev[i][hk][1])
            elif i % every == 1:
                ops.profile_kernel(0)
            step(i, timing=tim)
            step_ev[i + 1].record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        ops.profile_kernel(0)
    ms_per_step = (t1 - t0) * 1e3 / K
    for i, names in armed.items():
        for k in names:
            kernel_ms[k].append(kev[i][k][0].elapsed_time(kev[i][k][1]))
    step_ms = [step_ev[i].elapsed_time(step_ev[i + 1]) for i in range(K)]

    # the same kernels undisturbed: a few untimed steps with both classes on one stream
    alone_ms = {}
    if split or keyed:
        opt.one_stream = True
        aev = [{k: new_events(2) for k in knames} for _ in range(3)]
        for j in range(3):
            tim = {k: aev[j][k] for k in knames if k not in hook_of and k != "cold_refresh"}
            ops.profile_kernel(hook_of["seg_sum"], aev[j]["seg_sum"][0], aev[j]["seg_sum"][1])
            run_step(wl.ids[j % nb], wl.grads[j % nb], mode, None, tim)   # one batch at a time
        ops.profile_kernel(0)
        torch.cuda.synchronize()
        opt.one_stream = False
        pipe["i"] = None
        alone_ms = {k: sum(aev[j][k][0].elapsed_time(aev[j][k][1]) for j in range(3)) / 3
                    for k in knames if k != "cold_refresh"}

    # phases: a second, untimed pass with four event records per step on the main stream
    for i in range(K):
        step(i, events=phase_ev[i])
    torch.cuda.synchronize()
    phases = ("fetch", "combine", "update")
    phase_ms = {p: sum(phase_ev[i][k].elapsed_time(phase_ev[i][k + 1]) for i in range(K)) / K
                for k, p in enumerate(phases)}

    # distinct ids per step and hot-hit statistics of the batches actually used
    uniq, hot_q, uniq_hot = [], [], []
    for q in wl.ids:
        u = torch.unique(q)
        uniq.append(u.numel())
        if wl.H:
            hot_q.append(int((ops.lookup(q, opt.hot_ids) >= 0).sum()))
            uniq_hot.append(int((ops.lookup(u, opt.hot_ids) >= 0).sum()))
        else:
            hot_q.append(0)
            uniq_hot.append(0)
    U = sum(uniq) / len(uniq)
    U_hot = sum(uniq_hot) / len(uniq_hot)
    n_hot = sum(hot_q) / len(hot_q)
    n_cold, U_cold = n - n_hot, U - U_hot
    # Algorithmic bytes per launch (fp32; one launch covers the whole batch or its class).
    # fetch 16 + 8D per query row; segmented sum n(8+4D) read + U*4D written; Adagrad 8 + 20D per
    # distinct row.  A cold row moves 4D bytes over the host link in the fetch and 4D each way in
    # the update (weights; the cold Adagrad state sits in HBM).
    # (SparseAdam: 16 + 28D - the id, the step counter both ways, and g, mem, power, w read,
    # mem, power, w written.)
    row_f, row_u = 16 + 8 * D, (16 + 28 * D) if args.optimizer == "adam" else (8 + 20 * D)
    alg_bytes = {"fetch": n * row_f, "combine": n * (8 + 4 * D) + U * (16 + 4 * D), "update": U * row_u}
    kbytes = {"fetch": n * row_f, "update": U * row_u,
              "seg_sum": (n_hot * (8 + 4 * D) + U_hot * 4 * D) if keyed else (n * (8 + 4 * D) + U * 4 * D),
              "hot_fetch": n_hot * row_f, "cold_fetch": n_cold * row_f,
              "hot_update": U_hot * row_u, "cold_update": U_cold * row_u}
    traffic = measured_traffic(workload, args.mode)
    if args.optimizer != "adagrad":     # the committed counters are those of the Adagrad kernels
        traffic = {k: v for k, v in traffic.items() if "update" not in k}
    kernels = {}
    for k, name in knames.items():
        if not kernel_ms[k]:
            continue
        ms = sum(kernel_ms[k]) / len(kernel_ms[k])
        if k not in kbytes:     # no byte model: the time only
            kernels[k] = {"kernel": name, "us": round(ms * 1e3, 2), "launches_timed": len(kernel_ms[k]),
                          "bound": "latency"}
            continue
        gbs = kbytes[k] / (ms * 1e-3) / 1e9
        entry = {"kernel": name, "us": round(ms * 1e3, 2), "launches_timed": len(kernel_ms[k]),
                 "bytes_per_launch": int(kbytes[k]), "GB/s": round(gbs, 1)}
        if k in alone_ms:
            a_ms = alone_ms[k]
            entry["us_alone"] = round(a_ms * 1e3, 2)
            entry["GB/s_alone"] = round(kbytes[k] / (a_ms * 1e-3) / 1e9, 1)
            if not (k.startswith("cold_") and wl.host_cold):
                entry["frac_alone"] = round(kbytes[k] / (a_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
        if k.startswith("cold_") and wl.host_cold:
            entry["bound"] = "pcie"
        else:
            entry["bound"] = "hbm"
            entry["frac"] = round(gbs / HBM_PEAK_GBS, 4)
            tb = traffic.get(k)
            entry["traffic"] = tb
            if tb:
                entry["traffic_GB/s"] = round(tb / (ms * 1e-3) / 1e9, 1)
                entry["traffic_frac"] = round(tb / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
        kernels[k] = entry
    # the headline roofline: the HBM-bound row kernel that moves the most bytes (hot traffic)
    hbm_keys = [k for k in kernels if kernels[k]["bound"] == "hbm"]
    main_k = "hot_fetch" if "hot_fetch" in kernels else max(hbm_keys, key=lambda k: kbytes[k])
    mk = kernels[main_k]
    roofline = {"bound": "hbm", "kernel": mk["kernel"], "achieved": mk["GB/s"], "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": mk["frac"], "traffic": mk.get("traffic"),
                "traffic_source": ("profiles/%s_step_hbm_traffic.txt (rocprofv3 FETCH_SIZE + "
                                   "WRITE_SIZE of an earlier run of this command)" % workload)
                if mk.get("traffic") else None,
                "kernel_us": mk["us"], "launches_timed": "%d of the %d in the timed region" %
                (mk["launches_timed"], K) if schedule != "graph" else "eager steps before the timed region",
                "timing": "HIP events recorded on the launch stream right before and after the "
                          "launch: the kernel plus about 3 us of dispatch latency",
                "bytes_per_launch": mk["bytes_per_launch"],
                # achieved / frac price the kernel on its ALGORITHMIC bytes; where queries repeat,
                # part of those bytes is served by L2, so the rate of bytes that reached HBM
                # (counter traffic over the same time) is stated beside it and is the lower one
                "achieved_is": "algorithmic bytes per launch / kernel time",
                "traffic_GB/s": mk.get("traffic_GB/s"), "traffic_frac": mk.get("traffic_frac")}
    if wl.host_cold:
        roofline["step_bound"] = ("the step as a whole is bound by the host link, not by HBM: see "
                                  "`pcie` (this object is the HBM kernel that moves the most bytes)")
    if split or keyed:
        hot_b = sum(kbytes[k] for k in ("hot_fetch", "seg_sum", "hot_update"))
        hot_ms = sum(kernels[k]["us"] for k in ("hot_fetch", "seg_sum", "hot_update")) / 1e3
        roofline["hot_traffic_all_row_kernels"] = {
            "GB/s": round(hot_b / (hot_ms * 1e-3) / 1e9, 1),
            "frac": round(hot_b / (hot_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "note": "hot gather + segmented sum + hot update: algorithmic bytes over the sum of "
                    "their kernel times in the timed region, where the segmented sum and the hot "
                    "update run beside the cold update and slow down with it"}
        if alone_ms:
            a_ms = sum(alone_ms[k] for k in ("hot_fetch", "seg_sum", "hot_update"))
            roofline["hot_traffic_all_row_kernels"]["GB/s_alone"] = round(hot_b / (a_ms * 1e-3) / 1e9, 1)
            roofline["hot_traffic_all_row_kernels"]["frac_alone"] = round(
                hot_b / (a_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
            roofline["hot_traffic_all_row_kernels"]["alone_note"] = (
                "the same kernels in three untimed steps with both classes on one stream "
                "(nothing on the host link beside them)")
    if pipelined:   # the forward half runs on side streams: the main stream sees one phase
        tot = sum(phase_ms.values())
        phase_ms = {"backward of batch i + completion of batch i+1 (main stream)": tot}
        phase_bytes = {next(iter(phase_ms)): sum(alg_bytes.values())}
        phases = tuple(phase_ms)
    elif keyed:     # the sums are interleaved with the updates: one backward phase
        phase_ms = {"fetch": phase_ms["fetch"], "combine+update": phase_ms["combine"] + phase_ms["update"]}
        phase_bytes = {"fetch": alg_bytes["fetch"], "combine+update": alg_bytes["combine"] + alg_bytes["update"]}
        phases = tuple(phase_ms)
    else:
        phase_bytes = alg_bytes
    per_phase = {p: {"ms": round(phase_ms[p], 4),
                     "GB/s": round(phase_bytes[p] / (phase_ms[p] * 1e-3) / 1e9, 1),
                     "frac_hbm": round(phase_bytes[p] / (phase_ms[p] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
                 for p in phases}
    total_bytes = sum(alg_bytes.values())
    res = {"workload": wl.describe(), "schedule": schedule, "n": n,
           "ms_per_step": ms_per_step,
           "step_us": {"mean": round(ms_per_step * 1e3, 1),
                       "mean_by_events": round(sum(step_ms) / len(step_ms) * 1e3, 1),
                       "max": round(max(step_ms) * 1e3, 1),
                       "slow_steps": [(i, round(t * 1e3, 1)) for i, t in enumerate(step_ms)
                                      if t > 1.3 * pct(step_ms, 50)],
                       "median": round(pct(step_ms, 50) * 1e3, 1),
                       "p10": round(pct(step_ms, 10) * 1e3, 1), "p90": round(pct(step_ms, 90) * 1e3, 1),
                       "note": "mean: wall clock over the K timed steps; the rest: the same steps by HIP "
                               "events at the step boundaries (slow_steps: index and time of those "
                               "above 1.3 x the median)"},
           "roofline": roofline, "kernels": kernels,
           "phases": per_phase,
           "phases_note": "from a second, untimed pass with four event records per step (each adds "
                          "3-4 us to its phase)" +
                          ("; fetch = both gathers and the id sort that runs beside the cold one"
                           if split else "") +
                          ("; fetch = the forward half (lookup, partition, both gathers, sort of the "
                           "keys beside the cold gather); combine is inside update = the backward "
                           "half (cold sums, cold update beside hot sums and hot update)"
                           if keyed and not pipelined else ""),
           "step_alg_GB": round(total_bytes / 1e9, 4),
           "step_GB/s": round(total_bytes / (ms_per_step * 1e-3) / 1e9, 1),
           "step_frac_hbm": round(total_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
           "unique_per_step": round(U, 1), "unique_hot_per_step": round(U_hot, 1),
           "hot_hit": round(n_hot / n, 4), "parity_gate": gate}
    if wl.host_cold:
        def link_entry(rows, ms, read_rows=1, write_rows=0):
            """rows x (read_rows to the device, write_rows to the host) table rows of 4D bytes in
            ms; GB/s and fraction of nominal are those of the busier direction"""
            rd, wr = rows * read_rows * 4 * D, rows * write_rows * 4 * D
            gbs = max(rd, wr) / (ms * 1e-3) / 1e9
            e = {"MB": round(max(rd, wr) / 1e6, 2), "GB/s": round(gbs, 2),
                 "frac_nominal": round(gbs / PCIE_PEAK_GBS, 4)}
            if read_rows != write_rows and min(rd, wr) > 0:
                e["MB_to_device"], e["MB_to_host"] = round(rd / 1e6, 2), round(wr / 1e6, 2)
                e["GB/s_to_device"] = round(rd / (ms * 1e-3) / 1e9, 2)
                e["GB/s_to_host"] = round(wr / (ms * 1e-3) / 1e9, 2)
            return e, gbs
        pcie = {"bound": "pcie", "peak": PCIE_PEAK_GBS, "unit": "GB/s per direction",
                "cold_query_rows": round(n_cold, 1), "cold_unique_rows": round(U_cold, 1),
                "memcpy": link}
        write_only = keyed and reuse_rows and reused["no"] == 0 and reused["yes"] > 0
        # rows of 4D bytes per distinct cold row that the update reads / writes over the link
        soh = wl.state_on_host
        u_rd, u_wr = (1 if soh else 0) + (0 if write_only else 1), (2 if soh else 1)
        if split or keyed:
            f, f_gbs = link_entry(n_cold, kernels["cold_fetch"]["us"] / 1e3)
            u, u_gbs = link_entry(U_cold, kernels["cold_update"]["us"] / 1e3, u_rd, u_wr)
            timing_note = "cold-class kernels bracketed by HIP events on the cold stream"
        else:
            f, f_gbs = link_entry(n_cold, kernels["fetch"]["us"] / 1e3)
            u, u_gbs = link_entry(U_cold, kernels["update"]["us"] / 1e3, u_rd, u_wr)
            timing_note = "hot and cold rows share the kernels: kernel time of the whole fetch / update"
        if link:
            f["frac_memcpy_h2d"] = round(f_gbs / link["h2d_GB/s"], 4)
            u["frac_memcpy_h2d"] = round(u_gbs / link["h2d_GB/s"], 4)
            u["frac_memcpy_both_ways"] = round(u_gbs / link["both_ways_each_GB/s"], 4)
            if "kernels" in link:
                u["frac_kernel_probe_both_ways"] = round(u_gbs / link["kernels"]["both_ways_each_GB/s"], 4)
                f["frac_kernel_probe_gather"] = round(f_gbs / link["kernels"]["gather_GB/s"], 4)
        pcie["fetch_host_to_device"] = f
        if soh:
            pcie["update_state_on_host"] = u
            pcie["update_note"] = (
                "weights and Adagrad state of the cold rows are both in host memory, side by side: per "
                "distinct cold row the update reads %d B (%s) and writes %d B (new weight and state, "
                "one stretch) over the link" % (u_rd * 4 * D, "the state; the old weight comes from "
                "the rows this step fetched" if write_only else "weight and state", u_wr * 4 * D))
        elif write_only:
            pcie["update_device_to_host_only"] = u
            pcie["update_note"] = ("the cold update takes the old weights from the rows this step's "
                                   "fetch brought in (backward_keyed's guarded default: the optimizer "
                                   "saw no write to the table between the two halves in any of the "
                                   "%d backward halves of this run): it only writes over the link"
                                   % reused["yes"])
        else:
            pcie["update_each_way_at_once"] = u
        pcie["achieved"] = round(min(f_gbs, u_gbs), 2)
        pcie["frac"] = round(min(f_gbs, u_gbs) / PCIE_PEAK_GBS, 4)
        pcie["legs"] = {"fetch_host_to_device": round(f_gbs / PCIE_PEAK_GBS, 4),
                        ("update_state_on_host" if soh else
                         "update_device_to_host_only" if write_only else "update_each_way_at_once"):
                            round(u_gbs / PCIE_PEAK_GBS, 4)}
        pcie["note"] = ("%s; %s; achieved/frac = the lower of the two legs" % (
            timing_note, "the update's rate is that of its busier direction" if soh else
            "the update only writes the cold weight rows (4D bytes per distinct cold row)"
            if write_only else
            "the update reads and writes the cold weight rows (4D bytes each way per distinct cold row)"))
        res["pcie"] = pcie
    if keyed:
        res["backward_halves_that_reused_the_forward_rows"] = dict(reused)
    one_sweep = bool(ops._lib.query("hades_sort_mode"))
    res["sort"] = {"form": "one sweep: histogram of all digits, then one kernel per digit with bounded "
                           "look-back waits" if one_sweep else
                           "per digit a count kernel, a scan kernel for large batches and a scatter kernel"}
    if one_sweep and opt._ws.buf is not None:
        res["sort"]["tiles_whose_wait_ran_out_in_the_last_sort"] = ops.sort_wait_expiries(opt._ws)
    del wl, opt
    torch.cuda.empty_cache()
    return res


def run_cfg4(args):
    """Cold-gradient accumulator with a delayed write-back: every step combines a batch of cold
    ids and adds the distinct rows to the hash table in HBM; every `flush_every` steps the live
    entries leave the table in id order and go through sparse Adagrad on the pinned-host table.
    Prints its own JSON line (the step is not the headline fetch+combine+update step)."""
    import torch
    from hades_amd import ops, synth
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cfg = synth.CONFIGS["cfg4"]
    N, D, H, n = cfg["num_rows"], cfg["dim"], cfg["num_hot"], cfg["batch"]
    slots, every = cfg["num_slots"], cfg["flush_every"]
    seed = 1234 + 4
    nb = every
    log("allocating the %d x %d pinned host table (%.1f GB)" % (N, D, N * D * 4 / 1e9))
    cold_w = torch.empty((N, D), dtype=torch.float32, pin_memory=True)
    log("filling it")
    synth.fill_normal_(cold_w, 0.01, seed, progress=log)
    cold_s = torch.zeros((N, D), dtype=torch.float32, device=dev)
    log("sampling %d batches of %d cold ids" % (nb, n))
    # a Zipf law of its own over the cold ranks: cold rank k is global rank H + k
    sampler = synth.ZipfSampler(N - H, cfg["zipf_s"], dev)
    ids = [synth.make_ids(sampler, N, n, seed * 1000 + b, rank_offset=H) for b in range(nb)]
    grads = [synth.make_grads(n, D, seed * 2000 + b, dev) for b in range(nb)]
    del sampler
    acc = ops.ColdGradAccumulator(slots, D, id_bound=N, device=dev)
    ws = ops.Workspace(dev)
    comb_out = (torch.empty(n, dtype=torch.int64, device=dev),
                torch.empty((n, D), dtype=torch.float32, device=dev),
                torch.empty(n, dtype=torch.int64, device=dev),
                torch.empty(1, dtype=torch.int64, device=dev))
    cap = slots
    # The write-back of a flush runs on a side stream, beside the next steps' combine and
    # accumulate (it only touches the host table and the flushed rows): two sets of flush
    # buffers alternate, and a flush waits for the write-back that last read its set.
    # --schedule serial keeps it on the main stream.
    overlapped = args.schedule != "serial"
    from hades_amd.sparse_optim import side_stream
    wb_stream = side_stream(dev, 0)
    flush_sets = [(torch.empty(cap, dtype=torch.int64, device=dev),
                   torch.empty((cap, D), dtype=torch.float32, device=dev),
                   torch.empty(cap, dtype=torch.int64, device=dev),
                   torch.empty(1, dtype=torch.int64, device=dev)) for _ in range(2 if overlapped else 1)]
    wb_done = [None] * len(flush_sets)
    all_pos = torch.arange(cap, dtype=torch.int64, device=dev)
    wb_ev = []
    log("workload ready")

    def new_events(count):
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(count)]
        for e in evs:
            e.record()
        return evs

    ev = [new_events(5) for _ in range(args.steps)]
    kev = [new_events(2) for _ in range(args.steps)]
    live_at_flush = []

    def step(i, events=None):
        q, g = ids[i % nb], grads[i % nb]
        if events: events[0].record()
        uids, sums, cnts, nu = ops.combine_padded(q, g, id_bound=N, workspace=ws, out=comb_out)
        if events: events[1].record()
        acc.accumulate(uids, sums, cnts, num_rows=nu)
        if events: events[2].record()
        if (i + 1) % every == 0:
            k = ((i + 1) // every) % len(flush_sets)
            if wb_done[k] is not None:
                torch.cuda.current_stream().wait_event(wb_done[k])
            fi, fs, fc, fn = acc.flush_padded(cap, out=flush_sets[k])
            if events: events[3].record()
            if overlapped:
                flushed = torch.cuda.Event()
                flushed.record()
                wb_stream.wait_event(flushed)
                with torch.cuda.stream(wb_stream):
                    pair = new_events(2) if events else None
                    if pair: pair[0].record(wb_stream)
                    ops.adagrad_update_listed_(fi, fs, all_pos, fn, cold_w, cold_s, 0.01, 1e-10)
                    if pair:
                        pair[1].record(wb_stream)
                        wb_ev.append(pair)
                    wb_done[k] = torch.cuda.Event()
                    wb_done[k].record(wb_stream)
            else:
                ops.adagrad_update_(fi, fs, None, None, cold_w, cold_s, None, 0.01, 1e-10,
                                    num_unique=fn)
            if events: events[4].record()
            return fn
        return None

    warm = max(every, (args.warmup + every - 1) // every * every)   # ends on a flush
    for i in range(warm):
        step(i)
    torch.cuda.synchronize()
    assert int(acc.status.item()) == 0, "accumulator overflow during warm-up"
    log("warm-up of %d steps done" % warm)
    t0 = time.perf_counter()
    for i in range(args.steps):
        ops.profile_kernel(ops.KERNEL_HASH_ACCUMULATE, kev[i][0], kev[i][1])
        fn = step(i, ev[i])
        if fn is not None:
            live_at_flush.append(fn.clone())
    torch.cuda.synchronize()      # the last write-back included
    t1 = time.perf_counter()
    ops.profile_kernel(0)
    assert int(acc.status.item()) == 0, "accumulator overflow"
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    K = args.steps
    # the accumulate kernel undisturbed: every - 1 further steps (none of them flushes) with no
    # write-back in flight
    aev = [new_events(2) for _ in range(every - 1)]
    for j in range(every - 1):
        ops.profile_kernel(ops.KERNEL_HASH_ACCUMULATE, aev[j][0], aev[j][1])
        step(j)
    ops.profile_kernel(0)
    torch.cuda.synchronize()
    alone_ms = sum(a.elapsed_time(b) for a, b in aev) / max(1, len(aev))
    flush_steps = [i for i in range(K) if (i + 1) % every == 0]
    comb_ms = sum(ev[i][0].elapsed_time(ev[i][1]) for i in range(K)) / K
    acc_ms = sum(ev[i][1].elapsed_time(ev[i][2]) for i in range(K)) / K
    kern_ms = sum(kev[i][0].elapsed_time(kev[i][1]) for i in range(K)) / K
    U = sum(int(torch.unique(q).numel()) for q in ids) / nb
    live = [int(x.item()) for x in live_at_flush]
    L = sum(live) / max(1, len(live))
    line = {
        "metric": "cold gradient rows/s (combine + accumulate, flush + Adagrad write-back every %d steps)" % every,
        "value": round(n / (ms_per_step * 1e-3), 1), "unit": "rows/s", "n_gpus": 1,
        "steps": K, "warmup": warm, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "cfg4: %d cold ids/step zipf s=%.2f over ranks %d..%d of a %d x %d "
                               "pinned-host table, %d-slot accumulator in HBM, flush every %d steps"
                               % (n, cfg["zipf_s"], H + 1, N, N, D, slots, every)},
        "unique_per_step": round(U, 1), "live_keys_at_flush": round(L, 1),
        "load_at_flush": round(L / slots, 4),
        "phases": {"combine_ms": round(comb_ms, 4), "accumulate_ms": round(acc_ms, 4)},
    }
    # accumulate kernel: per distinct row 8 B id + 8 B count + 4D gradient read, 8 B key probe,
    # 8 B count and 4D accumulator read-modify-write (2 x 4D)
    kbytes = U * (16 + 4 * D + 8 + 16 + 8 * D)
    achieved = kbytes / (kern_ms * 1e-3) / 1e9
    alone = kbytes / (alone_ms * 1e-3) / 1e9
    line["roofline"] = {"bound": "hbm", "kernel": "hash_accumulate_kernel (hades_hash_accumulate)",
                        "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                        "kernel_us": round(kern_ms * 1e3, 2), "bytes_per_launch": int(kbytes),
                        "kernel_us_alone": round(alone_ms * 1e3, 2), "GB/s_alone": round(alone, 1),
                        "frac_alone": round(alone / HBM_PEAK_GBS, 4),
                        "note": "kernel_us: the launches of the timed steps, which run beside the "
                                "write-back of the previous flush when that is on the side stream "
                                "(HBM kernels slow down while requests to host memory are in flight); "
                                "alone: %d further steps after the timed region with nothing on the "
                                "host link" % (every - 1)}
    if flush_steps:
        fl_ms = sum(ev[i][2].elapsed_time(ev[i][3]) for i in flush_steps) / len(flush_steps)
        if overlapped:
            ap_ms = sum(a.elapsed_time(b) for a, b in wb_ev) / max(1, len(wb_ev))
            line["config"]["write_back"] = ("on a side stream beside the next steps (two sets of flush "
                                            "buffers); hades_adagrad_update_listed on 128 blocks")
        else:
            ap_ms = sum(ev[i][3].elapsed_time(ev[i][4]) for i in flush_steps) / len(flush_steps)
        line["phases"]["flush_ms_per_flush"] = round(fl_ms, 4)
        line["phases"]["apply_ms_per_flush"] = round(ap_ms, 4)
        # flush: scan of all keys, then per live entry key+count+row out of the table, row zeroed,
        # and id+count+row written
        fbytes = slots * 8 + L * (16 + 4 * D) * 2 + L * 4 * D
        line["flush_GB/s"] = round(fbytes / (fl_ms * 1e-3) / 1e9, 1)
        line["pcie"] = {"apply_read_GB/s": round(L * 4 * D / (ap_ms * 1e-3) / 1e9, 2),
                        "apply_write_GB/s": round(L * 4 * D / (ap_ms * 1e-3) / 1e9, 2),
                        "peak_per_direction": PCIE_PEAK_GBS}
    print(json.dumps(line))


def run_cfg4_staleness(args):
    """cfg4 with the reference's own rule instead of "every 8 steps": the cold-data cache of the
    cache server (set-associative index over 4 M slots, per-row staleness thresholds from the
    hotness, count threshold 16) in front of the pinned-host table.  Per step: combine the batch;
    gradients of cached ids accumulate in their slots; the other ids are applied to the host
    table at once and their rows enter the cache; rows that are due leave the cache and are
    applied.  No host synchronisation inside a step.  Prints its own JSON line."""
    import torch
    from hades_amd import ops, synth
    from hades_amd.cold_cache import ColdDataCache
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cfg = synth.CONFIGS["cfg4"]
    N, D, H, n, slots = cfg["num_rows"], cfg["dim"], cfg["num_hot"], cfg["batch"], cfg["num_slots"]
    seed = 1234 + 4
    warm = max(args.warmup, 8)
    # a fresh batch of ids for every step of the warm-up and of both measured passes: a cache sees
    # the stream's long tail only if the ids do not come round again; the gradient rows (268 MB a
    # batch) are reused
    nb, ng = warm + 2 * args.steps, 4
    log("allocating the %d x %d pinned host table (%.1f GB)" % (N, D, N * D * 4 / 1e9))
    cold_w = torch.empty((N, D), dtype=torch.float32, pin_memory=True)
    log("filling it")
    synth.fill_normal_(cold_w, 0.01, seed, progress=log)
    cold_s = torch.zeros((N, D), dtype=torch.float32, device=dev)
    log("sampling %d batches of %d cold ids" % (nb, n))
    sampler = synth.ZipfSampler(N - H, cfg["zipf_s"], dev)
    ids = [synth.make_ids(sampler, N, n, seed * 1000 + b, rank_offset=H) for b in range(nb)]
    grads = [synth.make_grads(n, D, seed * 2000 + b, dev) for b in range(ng)]
    # hotness of an id = its expected number of occurrences per step: popular cold rows may wait
    # one iteration, the long tail up to 100 (threshold = ceil(1 / (0.001 + hotness)), capped)
    ranks = torch.arange(1, N - H + 1, dtype=torch.float64, device=dev)
    p = ranks.pow_(-cfg["zipf_s"])
    p.div_(p.sum())
    hotness = torch.zeros(N, dtype=torch.float32, device=dev)
    hotness[synth.rank_to_id(torch.arange(H + 1, N + 1, dtype=torch.int64, device=dev), N)] = \
        (p * n).float()
    del ranks, p, sampler
    cache = ColdDataCache(slots, D, hotness, cnt_threshold=16, device=dev)
    del hotness
    ws = ops.Workspace(dev)
    comb_out = (torch.empty(n, dtype=torch.int64, device=dev),
                torch.empty((n, D), dtype=torch.float32, device=dev),
                torch.empty(n, dtype=torch.int64, device=dev),
                torch.empty(1, dtype=torch.int64, device=dev))
    fetched = torch.empty((n, D), dtype=torch.float32, device=dev)
    log("workload ready")
    stats = {"miss": 0, "hit": 0, "flushed": 0}

    positions = torch.arange(n, dtype=torch.int64, device=dev)
    minus_one = torch.full((n,), -1, dtype=torch.int64, device=dev)
    zero = torch.zeros(n, dtype=torch.int64, device=dev)
    split_ws = ops.Workspace(dev)

    def step(i, count=False):
        """No host synchronisation: the number of distinct ids stays on the device, the entries
        past it are given the id -1 (no cache line: every cache operator answers -1 for them and
        leaves them alone), and the uncached ids go through position lists with device counts."""
        q, g = ids[i], grads[i % ng]
        uids, sums, cnts, nu = ops.combine_padded(q, g, id_bound=N, workspace=ws, out=comb_out)
        live = positions < nu
        live_ids = torch.where(live, uids, minus_one)
        locs = cache.accumulate_gradients_cold_remote(live_ids, sums)      # cached ids: delayed
        miss = live & (locs < 0)
        _, _, miss_pos, counts = ops.split_padded(torch.where(miss, minus_one, zero), workspace=split_ws)
        # the uncached ids are applied at once; the update hands back the new rows (w_out), which
        # are the rows a trainer would pull next: no third crossing of the link for the cache
        ops.adagrad_update_listed_(uids, sums, miss_pos, counts[1:2], cold_w, cold_s, 0.01, 1e-10,
                                   w_out=fetched)
        cache.update_cache(torch.where(miss, uids, minus_one), fetched)
        f_ids, f_grads, f_cnts, f_num = cache.staled_gradients_remote_padded(slots)
        ops.adagrad_update_(f_ids, f_grads, None, None, cold_w, cold_s, None, 0.01, 1e-10,
                            num_unique=f_num)
        if count:
            m = int(counts[1].item())
            stats["miss"] += m; stats["hit"] += int(nu.item()) - m
            stats["flushed"] += int(f_num.item())

    for i in range(warm):
        step(i)
    torch.cuda.synchronize()
    log("warm-up done, %d entries cached" % cache.index.get_valid_entries_num())
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(warm + i)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    for i in range(args.steps):                     # as many steps again, counted (more host syncs)
        step(warm + args.steps + i, count=True)
    K = args.steps
    miss, hit, flushed = (stats[k] / K for k in ("miss", "hit", "flushed"))
    # rows over the host link: uncached ids are read and written (the update also returns the new
    # rows for the cache); flushed rows are read and written
    host_rows = miss * 2 + flushed * 2
    line = {
        "metric": "cold gradient rows/s (combine + cold-data cache with the staleness rule + write-back)",
        "value": round(n / (ms_per_step * 1e-3), 1), "unit": "rows/s", "n_gpus": 1, "steps": K,
        "warmup": warm, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "cfg4 with the cache server's rule: %d cold ids/step zipf s=%.2f, "
                               "%d-slot set-associative cold-data cache in HBM, per-row staleness "
                               "threshold from the hotness, count threshold 16, %d x %d pinned-host "
                               "table" % (n, cfg["zipf_s"], slots, N, D)},
        "distinct_per_step": round((miss + hit), 1), "cached_hits_per_step": round(hit, 1),
        "uncached_per_step": round(miss, 1), "flushed_rows_per_step": round(flushed, 1),
        "cache_entries": cache.index.get_valid_entries_num(),
        "host_link_rows_per_step": round(host_rows, 1),
        "host_link_GB/s_both_ways": round(host_rows * 4 * D / (ms_per_step * 1e-3) / 1e9, 2),
    }
    print(json.dumps(line))


def run_neighbours(args):
    """The operators either side of the step, each timed on its own over `steps` calls after
    `warmup` (wall clock around a synchronised loop, so launch overheads count): the pre-exchange
    bucketing of a cfg5-sized batch, and the set-associative index cache / cold-data cache with
    the staleness rule at cfg4's size.  Prints its own JSON line."""
    import torch
    from hades_amd import ops, synth
    from hades_amd.cold_cache import ColdDataCache
    from hades_amd.index_cache import IndexCache
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    K, W = args.steps, args.warmup

    def timed(fn, setup=None):
        for _ in range(W):
            if setup: setup()
            fn()
        torch.cuda.synchronize()
        total = 0.0
        for _ in range(K):
            if setup:
                setup()
                torch.cuda.synchronize()
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            total += time.perf_counter() - t0
        return total / K * 1e3

    out = {}
    # ---- pre-exchange bucketing: 1 M ids x 64 floats, 4 machines x 8 trainers ----
    cfg = synth.CONFIGS["cfg5"]
    N, D, n = cfg["num_rows"], cfg["dim"], cfg["batch"] * cfg["trainers"]
    sampler = synth.ZipfSampler(N, cfg["zipf_s"], dev)
    ids = synth.make_ids(sampler, N, n, 99)
    del sampler
    grad = synth.make_grads(n, D, 98, dev)
    cnt = torch.ones(n, dtype=torch.int64, device=dev)
    rp = torch.tensor([i * N // 4 for i in range(5)], dtype=torch.int64, device=dev)
    ws = ops.Workspace(dev)
    ms = timed(lambda: ops.bucket_by_owner(ids, grad, cnt, rp, 8, 32, workspace=ws))
    moved = n * (8 + 8 + 4 * D) * 2                       # ids, counts and rows read and written
    out["bucket_by_owner"] = {"rows": n, "dim": D, "owners": 32, "ms": round(ms, 4),
                              "rows/s": round(n / ms * 1e3, 1),
                              "GB/s": round(moved / ms / 1e6, 1),
                              "frac_hbm": round(moved / ms / 1e6 / HBM_PEAK_GBS, 4)}
    log("bucket_by_owner %.3f ms" % ms)
    del grad, cnt

    # ---- index cache: 4 M entries, 512 K-id batches of cold ids ----
    c4 = synth.CONFIGS["cfg4"]
    N4, H4, n4, D4 = c4["num_rows"], c4["num_hot"], c4["batch"], c4["dim"]
    sampler = synth.ZipfSampler(N4 - H4, c4["zipf_s"], dev)
    batches = [torch.unique(synth.make_ids(sampler, N4, n4, 500 + b, rank_offset=H4)) for b in range(4)]
    del sampler
    ic = IndexCache(c4["num_slots"], device=dev)
    state = {"b": 0}

    def nxt():
        state["b"] = (state["b"] + 1) % len(batches)
        return batches[state["b"]]
    u = sum(b.numel() for b in batches) / len(batches)
    ms_add = timed(lambda: ic.add(nxt()))
    ms_look = timed(lambda: ic.cudalookup(nxt()))
    ms_touch = timed(lambda: ic.lookup(nxt()))
    out["index_cache"] = {"entries": ic.get_capacity(), "ids_per_call": round(u, 1),
                          "valid_entries": ic.get_valid_entries_num(),
                          "add_ms": round(ms_add, 4), "cudalookup_ms": round(ms_look, 4),
                          "lookup_with_aging_ms": round(ms_touch, 4),
                          "cudalookup_ids/s": round(u / ms_look * 1e3, 1),
                          # per id: 8 B id + 64 B line + 8 B loc
                          "cudalookup_GB/s": round(u * 80 / ms_look / 1e6, 1)}
    log("index cache add %.3f lookup %.3f aging lookup %.3f ms" % (ms_add, ms_look, ms_touch))
    del ic

    # ---- cold-data cache: insert, accumulate and staleness flush at the same size ----
    hot = torch.rand(N4, device=dev) * 0.2               # thresholds between 5 and 100 iterations
    cc = ColdDataCache(c4["num_slots"], D4, hot, cnt_threshold=16)
    del hot
    rows = [synth.make_grads(b.numel(), D4, 700 + i, dev) for i, b in enumerate(batches)]

    def pair():
        state["b"] = (state["b"] + 1) % len(batches)
        return batches[state["b"]], rows[state["b"]]
    ms_ins = timed(lambda: cc.update_cache(*pair()))
    ms_acc = timed(lambda: cc.accumulate_gradients_cold_remote(*pair()))
    cap = c4["num_slots"]
    ms_flush = timed(lambda: cc.staled_gradients_remote_padded(cap),
                     setup=lambda: cc.accumulate_gradients_cold_remote(*pair()))
    out["cold_data_cache"] = {"slots": cc.num_slots, "dim": D4, "rows_per_call": round(u, 1),
                              "update_cache_ms": round(ms_ins, 4),
                              "accumulate_ms": round(ms_acc, 4),
                              "staleness_flush_ms": round(ms_flush, 4),
                              # per accumulated row: gradient read, slot row read and written
                              "accumulate_GB/s": round(u * 12 * D4 / ms_acc / 1e6, 1)}
    log("cold cache insert %.3f accumulate %.3f flush %.3f ms" % (ms_ins, ms_acc, ms_flush))
    line = {"metric": "neighbouring operators, ms per call", "unit": "ms", "n_gpus": 1,
            "steps": K, "warmup": W, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "bucket_by_owner on a cfg5 batch; index cache and cold-data "
                                   "cache at cfg4's size"}}
    line.update(out)
    print(json.dumps(line))


def run_random_rows(args):
    """The ceiling of the access pattern itself: rows that are distinct, random and 512 bytes
    long, in tables of 4 M rows (2.1 GB, the size of the cold-gradient accumulator), moved by the
    plain listed gather, the listed scatter and the listed Adagrad update.  No row is touched
    twice and no two rows share a DRAM page, so neither L2 nor the memory-side cache helps: this
    is what the segmented sum (gradient rows in sort order) and the accumulator (slot rows) can
    reach at best.  Prints its own JSON line."""
    import torch
    from hades_amd import ops
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    S, D, U = 4_194_304, 128, 353_000
    g = torch.Generator().manual_seed(3)
    slots = torch.randperm(S, generator=g)[:U].to(dev)
    pos = torch.arange(U, device=dev)
    cnt = torch.tensor([U], device=dev)
    grad = torch.randn((U, D), device=dev) * 1e-3
    w = torch.zeros((S, D), device=dev)
    st = torch.zeros((S, D), device=dev)
    out = torch.empty((U, D), device=dev)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        tot = 0.0
        for _ in range(args.steps):
            ev[0].record(); fn(); ev[1].record()
            torch.cuda.synchronize()
            tot += ev[0].elapsed_time(ev[1])
        return tot / args.steps

    res = {}
    for name, fn, nbytes in (
            ("gather (hades_fetch_listed)", lambda: ops.fetch_listed(w, slots, pos, cnt, out), U * (16 + 8 * D)),
            ("scatter (hades_set_listed)", lambda: ops.set_listed(grad, w, slots, pos, cnt), U * (16 + 8 * D)),
            ("Adagrad (hades_adagrad_update_listed)",
             lambda: ops.adagrad_update_listed_(slots, grad, pos, cnt, w, st, 0.01, 1e-10), U * (16 + 20 * D))):
        ms = timed(fn)
        res[name] = {"us": round(ms * 1e3, 1), "GB/s": round(nbytes / ms / 1e6, 1),
                     "frac_hbm": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
        log("%s: %.1f us" % (name, ms * 1e3))
    a = torch.empty(64 << 20, dtype=torch.float32, device=dev).normal_()
    b = torch.empty_like(a)
    ms = timed(lambda: b.copy_(a))
    res["plain 256 MiB device copy (torch)"] = {"us": round(ms * 1e3, 1), "GB/s": round(2 * a.numel() * 4 / ms / 1e6, 1),
                                                "frac_hbm": round(2 * a.numel() * 4 / ms / 1e6 / HBM_PEAK_GBS, 4)}
    print(json.dumps({"metric": "distinct random 512-byte rows of a 2.1 GB table, GB/s of algorithmic bytes",
                      "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
                      "dtype": "f32", "data": "synthetic",
                      "config": {"workload": "%d distinct random rows of %d x %d fp32 tables" % (U, S, D)},
                      "operators": res}))


def run_host_link(args):
    """What the host link gives kernels on this box: random distinct rows of a 56.8 GB page-locked
    table moved by the library's own listed kernels, swept over rows per launch, grid width and
    burst length, one way and both ways at once.  Columns (GB/s of the busier direction):
      gather          host -> HBM (hades_fetch_listed)
      scatter         HBM -> host (hades_set_listed)
      gather||scatter both at once, two kernels on two streams
      update rw       hades_adagrad_update_listed, state in HBM: reads and writes the weight row
      update wo       hades_adagrad_update_class with the old rows at hand: only writes it
      pair rw         weight and state row of an id side by side in the host table ([N, 2, D],
                      1 KB per id): reads both, writes both
      pair r1w2       the same with the old weight rows at hand: reads the state, writes both
    Burst 512 B = rows of 128 floats; 1 KB = the same memory viewed as rows of 256 floats.
    Prints one JSON line; the table goes to stderr."""
    import types
    import torch
    from hades_amd import ops, synth
    from hades_amd.sparse_optim import side_stream
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    N, D = synth.CONFIGS["cfg3"]["num_rows"], 128
    log("allocating the %d x %d pinned host table (%.1f GB) and as much state in HBM" % (N, D, N * D * 4 / 1e9))
    table = torch.empty((N, D), dtype=torch.float32, pin_memory=True)
    synth.fill_normal_(table, 0.01, 77, progress=log)
    state = torch.zeros((N, D), dtype=torch.float32, device=dev)
    wide = table.view(N // 2, 2 * D)              # 1 KB rows
    pair = table.view(N // 2, 2, D)               # [ids, (weight, state), D]
    s1, s2 = side_stream(dev, 0), side_stream(dev, 1)
    row_counts = [76_000, 300_000, 1_200_000, 2_300_000]
    widths = [16, 32, 64, 128, 256]
    gen = torch.Generator().manual_seed(5)
    results = []
    reps = 3

    def timed(fns):
        best = None
        for _ in range(reps):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for f in fns:
                f()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        return best

    def case(R, tab_rows):
        ids = torch.randperm(tab_rows, generator=gen)[:R].to(dev).sort().values
        pos = torch.arange(R, dtype=torch.int64, device=dev)
        cnt = torch.tensor([R], dtype=torch.int64, device=dev)
        plan = types.SimpleNamespace(
            uids=ids, num_unique=cnt, n=R, key_bits=40,
            class_split=torch.tensor([R, R], dtype=torch.int64, device=dev),
            first_pos=torch.arange(R, dtype=torch.int32, device=dev))
        return ids, pos, cnt, plan

    for R in row_counts:
        ids5, pos, cnt, plan5 = case(R, N)
        ids1, _, _, plan1 = case(R, N // 2)
        buf5 = torch.empty((R, D), dtype=torch.float32, device=dev)
        src5 = torch.empty((R, D), dtype=torch.float32, device=dev)
        buf1 = torch.empty((R, 2 * D), dtype=torch.float32, device=dev)
        src1 = torch.empty((R, 2 * D), dtype=torch.float32, device=dev)
        grad = torch.randn((R, D), device=dev) * 1e-3
        ops.fetch_listed(table, ids5, pos, cnt, src5)       # the scatters write back what is there
        ops.fetch_listed(wide, ids1, pos, cnt, src1)
        old_pair = torch.empty((R, D), dtype=torch.float32, device=dev)
        ops.fetch_listed(pair[:, 0], ids1, pos, cnt, old_pair)
        torch.cuda.synchronize()

        def on(stream, fn):
            def run():
                with torch.cuda.stream(stream):
                    fn()
            return run

        pats = {
            ("gather", 512): [on(s1, lambda: ops.fetch_listed(table, ids5, pos, cnt, buf5))],
            ("scatter", 512): [on(s2, lambda: ops.set_listed(src5, table, ids5, pos, cnt))],
            ("gather", 1024): [on(s1, lambda: ops.fetch_listed(wide, ids1, pos, cnt, buf1))],
            ("scatter", 1024): [on(s2, lambda: ops.set_listed(src1, wide, ids1, pos, cnt))],
            ("update rw", 512): [on(s1, lambda: ops.adagrad_update_listed_(ids5, grad, pos, cnt, table, state, 0.01, 1e-10))],
            ("update wo", 512): [on(s1, lambda: ops.adagrad_update_class_(plan5, grad, 0, table, state, 0.01, 1e-10,
                                                                       fetched_rows=src5))],
            ("pair rw", 1024): [on(s1, lambda: ops.adagrad_update_listed_(ids1, grad, pos, cnt, pair[:, 0], pair[:, 1],
                                                                       0.01, 1e-10))],
            ("pair r1w2", 1024): [on(s1, lambda: ops.adagrad_update_class_(plan1, grad, 0, pair[:, 0], pair[:, 1], 0.01,
                                                                        1e-10, fetched_rows=old_pair))],
        }
        pats[("gather||scatter", 512)] = pats[("gather", 512)] + pats[("scatter", 512)]
        pats[("gather||scatter", 1024)] = pats[("gather", 1024)] + pats[("scatter", 1024)]
        for B in widths:
            for use in (ops.LINK_COPY, ops.LINK_READ_WRITE, ops.LINK_WRITE_ONLY):
                ops.set_host_link_blocks(use, B)
            for burst in (512, 1024):
                row = {"rows": R, "burst_B": burst, "blocks": B}
                for (name, b), fns in pats.items():
                    if b == burst:
                        # bytes of the busier direction: one burst per row
                        row[name] = round(R * burst / timed(fns) / 1e9, 2)
                results.append(row)
                log(json.dumps(row))
        del buf5, src5, buf1, src1, grad, old_pair
    for use in (ops.LINK_COPY, ops.LINK_READ_WRITE, ops.LINK_WRITE_ONLY):
        ops.set_host_link_blocks(use, 0)
    cols = ["gather", "scatter", "gather||scatter", "update rw", "update wo", "pair rw", "pair r1w2"]
    print("%9s %6s %6s " % ("rows", "burst", "blocks") + " ".join("%16s" % c for c in cols), file=sys.stderr)
    for r in results:
        print("%9d %6d %6d " % (r["rows"], r["burst_B"], r["blocks"]) +
              " ".join("%16s" % ("%.2f" % r[c] if c in r else "-") for c in cols), file=sys.stderr)
    print(json.dumps({"metric": "host-link GB/s of the busier direction, random distinct rows of a pinned host table",
                      "unit": "GB/s", "n_gpus": 1, "dtype": "f32", "data": "synthetic",
                      "peak_nominal_per_direction": PCIE_PEAK_GBS,
                      "config": {"workload": "%d x %d fp32 page-locked table (%.1f GB); wall clock around one "
                                             "launch (or one pair of launches), best of %d" %
                                             (N, D, N * D * 4 / 1e9, reps)},
                      "rows": results}))


def run_cpu_baseline(wl_name, seconds):
    """The same step with the CPU oracle (torch CPU ops, all host threads), on a bounded sample:
    the benchmark's own batches at full table size when that fits the host, repeated for about
    `seconds`."""
    import torch
    from hades_amd import synth
    from oracle import hades_oracle as O
    cfg = synth.CONFIGS[wl_name]
    N, D, H = cfg["num_rows"], cfg["dim"], cfg["num_hot"]
    sample = "full %s step" % wl_name
    if N * D * 4 > 8 << 30:            # bound host memory: shrink the table, keep batch and skew
        scale = (8 << 30) / (N * D * 4)
        N, H = int(N * scale), int(H * scale)
        sample = "%s batch and skew on a table cut to %d rows" % (wl_name, N)
    seed = 1234 + int(wl_name[3:])
    n = cfg["batch"] * cfg.get("trainers", 1)
    cold_w = torch.empty((N, D))
    synth.fill_normal_(cold_w, 0.01, seed)
    cold_s = torch.zeros((N, D))
    hot_ids = synth.hot_ids(N, H) if H else torch.empty(0, dtype=torch.int64)
    hot_w, hot_s = cold_w[hot_ids].clone(), torch.zeros((hot_ids.numel(), D))
    sampler = synth.ZipfSampler(N, cfg["zipf_s"])
    q = synth.make_ids(sampler, N, n, seed * 1000)
    g = synth.make_grads(n, D, seed * 2000)
    O.torch_step(cold_w, cold_s, hot_w, hot_s, hot_ids, q, g, 0.01, 1e-10)   # warm-up
    times = []
    t_end = time.perf_counter() + seconds
    while time.perf_counter() < t_end or len(times) < 3:
        t0 = time.perf_counter()
        O.torch_step(cold_w, cold_s, hot_w, hot_s, hot_ids, q, g, 0.01, 1e-10)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": round(n / med, 1), "unit": "rows/s", "cores": torch.get_num_threads(),
            "kind": "port", "ms_per_step": round(med * 1e3, 3),
            "sample": "%s, %d repetitions, median; torch CPU ops (searchsorted, index, unique + "
                      "index_add_, addcmul/addcdiv)" % (sample, len(times))}


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the all-to-all "
              "gradient exchange is out of scope); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.workload == "cfg4":
        if args.flush_rule == "staleness":
            run_cfg4_staleness(args)
        else:
            run_cfg4(args)
        return
    if args.workload == "neighbours":
        run_neighbours(args)
        return
    if args.workload == "random-rows":
        run_random_rows(args)
        return
    if args.workload == "host-link":
        run_host_link(args)
        return
    if args.optimizer != "adagrad":
        if args.workload == "cfg1":
            print("cfg1 is the CPU reference case: it runs with the configurations' Adagrad only",
                  file=sys.stderr)
            sys.exit(2)
        # the secondary runs and the CPU baseline are those of the configurations' optimizer
        args.no_secondary = True
        args.no_cpu_baseline = True
    fallback = None
    try:
        res = run_gpu(args, args.workload, args.schedule, reuse_rows=args.reuse_rows,
                      state_on_host=args.cold_state == "host")
    except WorkloadSetupError as err:
        # a host that refuses the 56.8 GB page-locked table (or lacks the HBM): say so and measure
        # the all-HBM configuration instead of printing nothing
        msg = str(err)
        if args.workload != "cfg3":
            raise
        if not args.allow_fallback:
            print("bench.py: cfg3 could not be set up on this host (%s).  Nothing was measured; "
                  "--allow-fallback measures cfg2 instead and labels the line so." % msg,
                  file=sys.stderr)
            sys.exit(3)
        log("cfg3 could not be set up (%s): falling back to cfg2" % msg)
        import gc
        import torch
        gc.collect()
        torch.cuda.empty_cache()
        fallback = "cfg3 could not be allocated on this host (%s); this line is cfg2" % msg
        args.workload, args.schedule = "cfg2", None
        res = run_gpu(args, "cfg2", None)
    ms_per_step = res.pop("ms_per_step")
    n = res.pop("n")
    schedule = res.pop("schedule")
    line = {
        "metric": "embedding rows/s (fetch+combine+update)",
        "value": round(n / (ms_per_step * 1e-3), 1),
        "unit": "rows/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": res.pop("workload") + (
                       "; the cold update re-reads the table (--no-reuse-rows)"
                       if (schedule in ("keyed", "pipelined") and not args.reuse_rows) else ""),
                   "combine_mode": args.mode,
                   "optimizer": ("SparseAdam lr=0.01 betas=(0.9, 0.999) eps=1e-8 (the reference's "
                                 "optimizer; the configurations name Adagrad)" if args.optimizer == "adam"
                                 else "sparse Adagrad lr=0.01 eps=1e-10"),
                   "duplicate_ids": {None: "the update applies the SUM of an id's gradient rows",
                                     "sum": "the update applies the SUM of an id's gradient rows",
                                     "mean": "the update applies the MEAN of an id's gradient rows, as the "
                                             "reference's update does (unique_grads)",
                                     "one_plus": "the update applies the sum of an id's gradient rows over "
                                                 "one plus its occurrences"}[
                       args.average if args.average is not None else
                       ("mean" if args.optimizer == "adam" else None)],
                   "schedule": {"serial": "one stream, hot and cold rows in the same kernels",
                                "split": "lookup + hot/cold partition; hot rows on the main stream, "
                                         "cold rows on a second stream of the same priority",
                                "keyed": "one lookup + hot/cold partition per batch; hot rows on the "
                                         "main stream, cold rows on a second stream of the same "
                                         "priority; combine over class-ordered keys: the cold class "
                                         "is summed first and its update overlaps the hot class",
                                "pipelined": "the keyed kernels with two batches in flight: the next "
                                             "batch's lookup, partition, cold gather and key sort run on "
                                             "side streams while this batch's cold update writes the host "
                                             "table; afterwards the cold rows that update wrote are read "
                                             "again, so every batch gets the rows and leaves the tables of "
                                             "the one-batch-at-a-time order, bit for bit (the trainer must "
                                             "know a batch's ids one step ahead)",
                                "overlap": "one stream + the sort of the step's ids on a side stream, "
                                           "concurrent with its fetch",
                                "graph": "one stream, every step replayed from a HIP graph captured "
                                         "once per batch"}[schedule]},
    }
    line.update(res)
    if fallback:
        line["config"]["fallback"] = fallback
    if args.workload == "cfg3" and not args.no_secondary:
        line["secondary"] = {}

        def secondary(key, what, build, **run_kw):
            """One nested measurement.  A host or GPU that cannot hold it (allocation refused) leaves
            a `skipped` entry instead of taking the headline down with it; a parity-gate failure is
            not caught."""
            log("secondary: " + key)
            try:
                sec = run_gpu(args, **run_kw)
            except (RuntimeError, MemoryError) as err:
                line["secondary"][key] = {"skipped": str(err).splitlines()[0][:300] if str(err)
                                          else type(err).__name__}
                import gc
                import torch
                gc.collect()
                torch.cuda.empty_cache()
                return
            entry = {"what": what} if what else {}
            entry.update(build(sec))
            line["secondary"][key] = entry

        def brief(sec):
            return {"value": round(sec["n"] / (sec["ms_per_step"] * 1e-3), 1), "unit": "rows/s",
                    "step_us": sec["step_us"], "phases": sec["phases"], "pcie": sec.get("pcie"),
                    "kernels": {k: {a: b for a, b in v.items() if a in ("us", "us_alone", "GB/s")}
                                for k, v in sec["kernels"].items()},
                    "parity_gate": sec["parity_gate"]}

        secondary("cfg2", None, lambda sec: {
            "workload": sec["workload"], "schedule": sec["schedule"],
            "value": round(sec["n"] / (sec["ms_per_step"] * 1e-3), 1), "unit": "rows/s",
            "step_us": sec["step_us"], "step_frac_hbm": sec["step_frac_hbm"],
            "roofline": sec["roofline"], "kernels": sec["kernels"], "phases": sec["phases"]},
            workload="cfg2", schedule=None, with_gate=False, with_link=False)
        if schedule == "keyed" and args.reuse_rows:
            secondary("cfg3_table_reread",
                      "the headline workload and schedule, but the cold update reads the old weight "
                      "rows from the host table a second time (backward_keyed(fetched_rows=None), or "
                      "an optimizer constructed with reuse_fetched_rows=False): what a table with "
                      "writers the optimizer cannot see has to do.  Bit-identical results", brief,
                      workload="cfg3", schedule="keyed", with_gate=True, with_link=False, reuse_rows=False)
        if schedule == "keyed" and args.reuse_rows and args.cold_state == "hbm":
            secondary("cfg3_cold_state_in_host_memory",
                      "the contract layout of the cold class: weights AND Adagrad state of the cold "
                      "rows in pinned host memory, the two rows of an id side by side ([N, 2, D], "
                      "1 KB per id), on a table cut to 55.5 M rows with 5.55 M hot so that the one "
                      "page-locked allocation this box grants (56.8 GB) holds both; cfg3's batch "
                      "size, skew and 10 % hot fraction",
                      lambda sec: dict(brief(sec), workload=sec["workload"], hot_hit=sec["hot_hit"],
                                       unique_per_step=sec["unique_per_step"]),
                      workload="cfg3", schedule="keyed", with_gate=True, with_link=False, reuse_rows=True,
                      state_on_host=True)
        if schedule == "keyed" and args.reuse_rows:
            from hades_amd import ops as _ops
            width = _ops.set_host_link_blocks(_ops.LINK_WRITE_ONLY, 34)
            try:
                secondary("cfg3_update_34_blocks",
                          "the headline workload and schedule with the write-only cold update 34 "
                          "workgroups wide instead of %d: the update gives up some of its link rate, "
                          "the hot-class sums and update beside it are slowed less - both of the "
                          "targets (hot-cache traffic at 60 %% of HBM peak inside the step, cold rows "
                          "at 70 %% of the link) are met in one and the same step, which is a few "
                          "per cent longer" % width,
                          lambda sec: dict(brief(sec), hot_traffic_all_row_kernels=sec["roofline"].get(
                              "hot_traffic_all_row_kernels")),
                          workload="cfg3", schedule="keyed", with_gate=True, with_link=False, reuse_rows=True)
            finally:
                _ops.set_host_link_blocks(_ops.LINK_WRITE_ONLY, width)
            secondary("cfg3_pipelined",
                      "the headline workload with the next batch's forward half (lookup, partition, "
                      "cold gather, key sort) running on side streams while this batch's cold update "
                      "writes the host table, so that the link carries reads and writes at once; the "
                      "cold rows that update wrote are read again afterwards, and every batch gets the "
                      "rows and leaves the tables of the one-batch-at-a-time order, bit for bit.  Needs "
                      "the ids of a batch one step ahead (prefetch_keyed / finish_prefetch) and, for the "
                      "reuse of the fetched rows, one writer per table row", brief,
                      workload="cfg3", schedule="pipelined", with_gate=True, with_link=False, reuse_rows=True)
    if not args.no_cpu_baseline:
        try:
            line["cpu_baseline"] = run_cpu_baseline(args.workload, args.cpu_seconds)
        except (RuntimeError, MemoryError) as err:
            line["cpu_baseline"] = {"value": None, "unit": "rows/s", "cores": None, "kind": "port",
                                    "sample": "not measured: %s" % (str(err).splitlines()[0][:200]
                                                                    if str(err) else type(err).__name__)}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
