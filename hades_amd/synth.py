"""Seeded synthetic workloads of the embedding-cache hot path (used by bench.py and the tests).

IDs follow a bounded Zipf law over ranks 1..N (p_k proportional to k^-s), sampled by inverse CDF
on a float64 cumulative table; ranks map to node ids by the fixed bijection
id = (a*(rank-1) + b) mod N with gcd(a, N) = 1, so hot ids are scattered over the id space; the
hot set is the ids of ranks 1..H, ascending.  Tables are float32 N(0, 0.01), gradients float32
N(0, 1e-3), one row per query.
"""
import math

import torch

# name -> (N, D, H, n per step, zipf s)
CONFIGS = {
    "cfg1": dict(num_rows=1_000_000, dim=64, num_hot=100_000, batch=65_536, zipf_s=1.1),
    "cfg2": dict(num_rows=2_400_000, dim=128, num_hot=480_000, batch=200_000, zipf_s=1.0),
    "cfg3": dict(num_rows=111_000_000, dim=128, num_hot=11_100_000, batch=1_000_000, zipf_s=1.05),
    "cfg4": dict(num_rows=111_000_000, dim=128, num_hot=11_100_000, batch=524_288, zipf_s=0.9,
                 num_slots=4_194_304, flush_every=8),
    "cfg5": dict(num_rows=244_000_000, dim=64, num_hot=0, batch=262_144, zipf_s=1.1, trainers=4),
}


def _bijection(num_rows):
    """(a, b) of the rank -> id map; a is the first integer >= 0.618*N coprime with N."""
    a = max(1, int(num_rows * 0.6180339887))
    while math.gcd(a, num_rows) != 1:
        a += 1
    return a, (num_rows // 3) % num_rows


def rank_to_id(rank, num_rows):
    """rank in [1, N] (int64 tensor) -> node id in [0, N)."""
    a, b = _bijection(num_rows)
    return ((rank - 1) * a + b) % num_rows


class ZipfSampler:
    """Bounded Zipf over `support` ranks, optionally offset (ranks first_rank..first_rank+support-1
    keep their global weights k^-s: used for the cold-only stream of the accumulator workload)."""

    def __init__(self, support, s, device="cpu", first_rank=1):
        self.support, self.first_rank = int(support), int(first_rank)
        self.device = torch.device(device)
        k = torch.arange(first_rank, first_rank + support, dtype=torch.float64, device=self.device)
        cdf = k.pow_(-float(s)).cumsum_(0)
        self.cdf = cdf.div_(cdf[-1].clone())

    def sample_ranks(self, n, generator):
        u = torch.rand(n, dtype=torch.float64, generator=generator).to(self.device)
        r = torch.searchsorted(self.cdf, u, right=False).clamp_(max=self.support - 1)
        return r + self.first_rank


def hot_ids(num_rows, num_hot, device="cpu"):
    """ids of ranks 1..H, ascending (int64)."""
    ranks = torch.arange(1, num_hot + 1, dtype=torch.int64, device=device)
    return torch.sort(rank_to_id(ranks, num_rows)).values


def make_ids(sampler, num_rows, n, seed, rank_offset=0):
    """n ids drawn from the sampler's ranks; rank_offset shifts them (H: a Zipf law of its own
    over the cold ranks H+1..N)."""
    g = torch.Generator().manual_seed(seed)
    return rank_to_id(sampler.sample_ranks(n, g) + rank_offset, num_rows)


def make_grads(n, dim, seed, device="cpu"):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(n, dim, generator=g, dtype=torch.float32) * 1e-3).to(device)


def fill_normal_(t, std, seed, chunk_rows=1 << 20, progress=None):
    """In-place N(0, std) fill, chunk-wise so that pinned host tables of tens of GB can be filled
    from the device without a second full-size buffer."""
    if t.is_cuda:
        g = torch.Generator(device=t.device).manual_seed(seed)
        for r0 in range(0, t.size(0), chunk_rows * 16):
            t[r0:r0 + chunk_rows * 16].normal_(0.0, std, generator=g)
        return t
    if torch.cuda.is_available():
        dev = torch.device("cuda")
        g = torch.Generator(device=dev).manual_seed(seed)
        buf = torch.empty((chunk_rows,) + tuple(t.shape[1:]), dtype=t.dtype, device=dev)
        for k, r0 in enumerate(range(0, t.size(0), chunk_rows)):
            rows = min(chunk_rows, t.size(0) - r0)
            buf[:rows].normal_(0.0, std, generator=g)
            t[r0:r0 + rows].copy_(buf[:rows])
            if progress and k % 16 == 15:
                progress("filled %d of %d rows" % (r0 + rows, t.size(0)))
        return t
    g = torch.Generator().manual_seed(seed)
    return t.normal_(0.0, std, generator=g)


def fill_interleaved_(t, std, seed, chunk_rows=1 << 19, progress=None):
    """In place, for a pinned host table [N, 2, D] that keeps the weight row and the optimizer
    state row of an id next to each other: t[:, 0] = N(0, std), t[:, 1] = 0.  Filled from the
    device in contiguous chunks (a strided host view would be copied through a CPU staging pass)."""
    assert t.dim() == 3 and t.size(1) == 2 and t.is_contiguous()
    if not torch.cuda.is_available() or t.is_cuda:
        g = torch.Generator(device=t.device).manual_seed(seed)
        t[:, 0].normal_(0.0, std, generator=g)
        t[:, 1].zero_()
        return t
    dev = torch.device("cuda")
    g = torch.Generator(device=dev).manual_seed(seed)
    buf = torch.zeros((chunk_rows,) + tuple(t.shape[1:]), dtype=t.dtype, device=dev)
    for k, r0 in enumerate(range(0, t.size(0), chunk_rows)):
        rows = min(chunk_rows, t.size(0) - r0)
        buf[:rows, 0].normal_(0.0, std, generator=g)
        t[r0:r0 + rows].copy_(buf[:rows])
        if progress and k % 32 == 31:
            progress("filled %d of %d rows" % (r0 + rows, t.size(0)))
    return t
