"""Shared-memory layer (host only, no GPU): segments are visible across processes, tensors over
them alias the mapping, the pool follows the reference's allocation policy
(python/EmbCache/base.py:36-111), and failures come back as exceptions with nothing left behind."""
import multiprocessing as mp
import os

import pytest
import torch

from hades_amd import shm

PREFIX = "hades_test_%d_" % os.getpid()


def _child_reads_and_writes(name, size, q):
    # a second process: open the creator's segment, check its contents, write an answer
    from hades_amd import shm as s
    ptr, fd = s.open_shared_mem(name, size, pin_memory=False)
    t = s.open_shared_tensor(ptr, torch.int64, (size // 8,))
    ok = bool((t[:100] == torch.arange(100)).all())
    t[100:200] = torch.arange(100) * 3
    os.close(fd)                      # leave the segment linked for the parent
    q.put(ok)


def test_segment_is_shared_between_processes():
    name, size = PREFIX + "a", 1 << 16
    ptr, fd = shm.create_shared_mem(name, size, pin_memory=False)
    try:
        assert shm.shared_mem_exists(name)
        t = shm.open_shared_tensor(ptr, "int64", (size // 8,))
        t.zero_()
        t[:100] = torch.arange(100)
        ctx = mp.get_context("spawn")
        q = ctx.Queue()
        p = ctx.Process(target=_child_reads_and_writes, args=(name, size, q))
        p.start()
        assert q.get(timeout=120) is True
        p.join(120)
        assert p.exitcode == 0
        assert torch.equal(t[100:200], torch.arange(100) * 3)
        del t
    finally:
        shm.release_shared_mem(name, size, ptr, fd, pin_memory=False)
    assert not shm.shared_mem_exists(name)


def test_open_errors_raise_and_leave_nothing():
    with pytest.raises(RuntimeError, match="fail to open"):
        shm.open_shared_mem(PREFIX + "missing", 4096, pin_memory=False)
    name = PREFIX + "b"
    ptr, fd = shm.create_shared_mem(name, 4096, pin_memory=False)
    try:
        with pytest.raises(RuntimeError, match="fewer than"):
            shm.open_shared_mem(name, 1 << 20, pin_memory=False)     # larger than the segment
        with pytest.raises(RuntimeError, match="size must be > 0"):
            shm.create_shared_mem(PREFIX + "zero", 0, pin_memory=False)
    finally:
        shm.release_shared_mem(name, 4096, ptr, fd, pin_memory=False)
    assert not shm.shared_mem_exists(name) and not shm.shared_mem_exists(PREFIX + "zero")


@pytest.mark.skipif(torch.cuda.is_available(), reason="exercises the no-device error path")
def test_pinning_failure_is_an_exception_not_an_exit():
    # without a device the runtime cannot register the mapping: the reference would exit here
    name = PREFIX + "pin"
    with pytest.raises(RuntimeError, match="cannot register"):
        shm.create_shared_mem(name, 4096, pin_memory=True)
    assert not shm.shared_mem_exists(name)


def test_pool_allocation_policy():
    pool = shm.ShmTensorPool(pin_memory=False)
    try:
        assert pool.create(PREFIX + "t", "float32", (0, 8)) is None            # base.py:43-44
        a = pool.create(PREFIX + "t", "float32", (100, 8))
        m1 = pool.meta(PREFIX + "t")
        assert m1.shm_size == int(100 * 8 * 4 * 1.2) and m1.shm_name == PREFIX + "t0"
        a.fill_(7.0)
        b = pool.create(PREFIX + "t", torch.float32, (110, 8))                  # fits: same segment
        m2 = pool.meta(PREFIX + "t")
        assert (m2.shm_name, m2.ptr, m2.shm_size) == (m1.shm_name, m1.ptr, m1.shm_size)
        assert m2.shape == (110, 8) and bool((b[:100] == 7.0).all())           # aliases the old rows
        del a, b
        c = pool.create(PREFIX + "t", torch.float32, (200, 8))                  # outgrown: new segment
        m3 = pool.meta(PREFIX + "t")
        assert m3.shm_name == PREFIX + "t1" and m3.shm_size == int(200 * 8 * 4 * 1.2)
        assert not shm.shared_mem_exists(m1.shm_name) and shm.shared_mem_exists(m3.shm_name)
        c.zero_()
        # a peer pool opens the same tensor by segment name
        peer = shm.ShmTensorPool(pin_memory=False)
        d = peer.open("remote", m3.shm_name, m3.shm_size, torch.float32, (200, 8))
        c[5, 3] = 2.5
        assert float(d[5, 3]) == 2.5
        assert peer.open("remote", m3.shm_name, m3.shm_size, torch.float32, (100, 16)).shape == (100, 16)
        assert peer.meta("remote").ptr == peer._shm_tensor_meta["remote"].ptr
        del c, d
        # the peer only unmaps in this test (a release would unlink the owner's segment)
        meta = peer._shm_tensor_meta.pop("remote")
        os.close(meta.fd)
        pool.release(PREFIX + "t")
        assert not shm.shared_mem_exists(m3.shm_name)
    finally:
        pool.close()


def test_dropin_module_exposes_the_shm_functions():
    import hades_amd.EmbCacheLib as E
    for name in ("create_shared_mem", "open_shared_mem", "release_shared_mem", "open_shared_tensor"):
        assert getattr(E, name) is getattr(shm, name)
