"""hades_combine_static (the entry point that allocates nothing: its scratch is a fixed array
inside the library) against hades_combine with a caller's workspace, through the C ABI.

Collected last on purpose (file name): it must pass both alone in a fresh process, where it makes
the first use of the library's scratch array, and after every other test."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _outs(n, dim):
    return (torch.empty(n, dtype=torch.int64, device="cuda"),
            torch.empty((n, dim), dtype=torch.float32, device="cuda"),
            torch.empty(n, dtype=torch.int64, device="cuda"),
            torch.full((1,), -7, dtype=torch.int64, device="cuda"),
            torch.empty(n, dtype=torch.int32, device="cuda"))


def _both(lib, idx, grad, bound, mode):
    """(static result, workspace result) of one batch, each trimmed to its number of distinct ids."""
    from hades_amd import _lib
    n, dim = idx.numel(), grad.size(1)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    a, b = _outs(n, dim), _outs(n, dim)
    _lib.call("hades_combine_static", _p(idx), _p(grad), n, dim, bound, mode,
              _p(a[0]), _p(a[1]), _p(a[2]), _p(a[3]), _p(a[4]), st)
    nbytes = _lib.query("hades_combine_workspace_bytes", n, dim)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    _lib.call("hades_combine", _p(idx), _p(grad), n, dim, bound, mode,
              _p(b[0]), _p(b[1]), _p(b[2]), _p(b[3]), _p(b[4]), _p(ws), nbytes, st)
    torch.cuda.synchronize()
    return a, b


def _same(a, b, n):
    ua, ub = int(a[3].item()), int(b[3].item())
    assert ua == ub and 0 < ua <= n
    for k in range(3):
        assert torch.equal(a[k][:ua], b[k][:ub]), k        # uids, sums (bit-exact), counts
    assert torch.equal(a[4], b[4])                          # inverse


@pytest.mark.parametrize("mode", [0, 1])                    # HADES_COMBINE_FAST, HADES_COMBINE_EXACT
def test_combine_static_matches_combine_twice_second_smaller(cuda_device, mode):
    rng = np.random.default_rng(2025 + mode)
    space, dim = 2_400_000, 128
    # first call: a large batch with long runs; second call: a smaller one that leaves most of the
    # scratch array holding the first call's tables
    for n in (200_000, 4_097):
        idx = np.minimum(rng.pareto(0.9, n).astype(np.int64) * 7919 % space, space - 1)
        grad = (rng.standard_normal((n, dim)) * 1e-3).astype(np.float32)
        t_idx, t_grad = torch.from_numpy(idx).cuda(), torch.from_numpy(grad).cuda()
        a, b = _both(None, t_idx, t_grad, space, mode)
        _same(a, b, n)
        if n < 10_000:      # and against the CPU oracle where that takes no time
            from oracle import hades_oracle as O
            wu, wsum, wc = O.combine_sequential(idx, grad)
            U = int(a[3].item())
            assert np.array_equal(a[0][:U].cpu().numpy(), wu)
            assert np.array_equal(a[2][:U].cpu().numpy(), wc)
            if mode == 1:
                assert np.array_equal(a[1][:U].cpu().numpy(), wsum)


def test_combine_static_limits_and_bound_flag(cuda_device):
    from hades_amd import _lib, ops
    lib = _lib.load()
    # a batch that needs more scratch than the library holds is refused, nothing is launched
    n, dim = 1_000_000, 128
    assert _lib.query("hades_combine_workspace_bytes_min", n, dim) > _lib.COMBINE_STATIC_SCRATCH_BYTES
    rc = lib.hades_combine_static(None, None, n, dim, 0, 0, None, None, None, None, None, None)
    assert rc == 1 and b"scratch" in lib.hades_last_error()
    # the largest single-trainer batch of the benchmark configurations fits
    assert _lib.query("hades_combine_workspace_bytes_min", 262_144, 128) <= _lib.COMBINE_STATIC_SCRATCH_BYTES
    # an id beyond id_bound: -1 distinct ids on this call, and no trace of it on the next one
    idx = torch.arange(5000, dtype=torch.int64, device="cuda") % 100
    grad = torch.ones((5000, 8), device="cuda")
    bad = idx.clone()
    bad[4321] = 100
    assert int(ops.combine_static(bad, grad, id_bound=100)[3].item()) == -1
    uids, sums, cnts, nu = ops.combine_static(idx, grad, id_bound=100)
    assert int(nu.item()) == 100 and torch.equal(cnts[:100], torch.full((100,), 50, device="cuda"))
    assert torch.equal(sums[:100], torch.full((100, 8), 50.0, device="cuda"))
    # empty batch
    e = ops.combine_static(idx[:0], grad[:0], id_bound=100)
    assert int(e[3].item()) == 0
