"""Shared-memory tensors: the host-side layer the reference's cache server and clients exchange
tables and buffers through.

Module functions keep the names and signatures of the reference's extension functions
(create_shared_mem / open_shared_mem / release_shared_mem / open_shared_tensor,
src/pybind.cc:38-45 over src/shm/shared_memory.h:14-66); `ShmTensorPool` keeps the bookkeeping of
EmbCacheBase (python/EmbCache/base.py:24-119): named tensors backed by segments allocated with
1.2x headroom (SHM_ALLOC_AMPL_TIMES, python/EmbCache/common.py:7), reused while they fit and
reallocated under a fresh segment name when they do not.

pin_memory=True registers the mapping with the HIP runtime, as the reference does with
cudaHostRegister.  Platforms that refuse to register existing memory make that raise; allocate
kernel-visible host tables with `EmbCacheLib.pinned_empty` there and keep shared segments for the
host-side exchange.
"""
import ctypes
from collections import namedtuple

import torch

from . import _lib

TensorMeta = namedtuple("TensorMeta", ["shm_name", "fd", "ptr", "shm_size", "dtype", "shape"])
SHM_ALLOC_AMPL_TIMES = 1.2          # python/EmbCache/common.py:7

_DTYPES = {"int32": torch.int32, "int64": torch.int64, "float32": torch.float32,
           "float64": torch.float64, "bool": torch.bool}          # common.py:24-34
_SIZEOF = {torch.int32: 4, torch.int64: 8, torch.float32: 4, torch.float64: 8, torch.bool: 1}


def str2dtype(name):
    return _DTYPES.get(name)


def dtype_sizeof(dtype):
    return _SIZEOF.get(_DTYPES.get(dtype, dtype) if isinstance(dtype, str) else dtype)


def _map(entry, name, size, pin_memory):
    ptr, fd = ctypes.c_void_p(), ctypes.c_int64()
    _lib.call(entry, name.encode(), int(size), 1 if pin_memory else 0, ctypes.byref(ptr),
              ctypes.byref(fd))
    return int(ptr.value), int(fd.value)


def create_shared_mem(name, size, pin_memory=True):
    """(ptr, fd) of a new segment of `size` bytes (src/shm/shared_memory.h:14-32)."""
    return _map("hades_shm_create", name, size, pin_memory)


def open_shared_mem(name, size, pin_memory=True):
    """(ptr, fd) of an existing segment (src/shm/shared_memory.h:34-48)."""
    return _map("hades_shm_open", name, size, pin_memory)


def release_shared_mem(name, size, ptr, fd, pin_memory=True):
    """Unregisters, unmaps, closes and unlinks (src/shm/shared_memory.h:50-58).  Tensors opened
    over the segment must not be used afterwards."""
    _lib.call("hades_shm_release", name.encode(), int(size), ctypes.c_void_p(ptr), int(fd),
              1 if pin_memory else 0)


def shared_mem_exists(name):
    """SharedMemory::Exist (src/shm/shared_memory.h:104-112)."""
    return bool(_lib.load().hades_shm_exists(name.encode()))


def open_shared_tensor(ptr, dtype, shape):
    """A tensor over mapped memory, without a copy (torch::from_blob in the reference,
    src/shm/shared_memory.h:60-66).  The caller keeps the mapping alive."""
    if isinstance(dtype, str):
        dtype = str2dtype(dtype)
    numel = 1
    for d in shape:
        numel *= int(d)
    nbytes = numel * dtype_sizeof(dtype)
    if nbytes == 0:
        return torch.empty(tuple(shape), dtype=dtype)
    buf = (ctypes.c_char * nbytes).from_address(int(ptr))
    return torch.frombuffer(buf, dtype=dtype, count=numel).view(tuple(int(d) for d in shape))


class ShmTensorPool:
    """Named shared tensors with the allocation policy of EmbCacheBase
    (python/EmbCache/base.py:24-119)."""

    def __init__(self, pin_memory=False):
        self._shm_tensor_meta = {}
        self._create_tensor_count = 0
        self._pin_memory = pin_memory

    def _create_shm_name(self, tensor_name):                       # base.py:31-34
        shm_name = tensor_name + str(self._create_tensor_count)
        self._create_tensor_count += 1
        return shm_name

    def meta(self, tensor_name):
        return self._shm_tensor_meta[tensor_name]

    def create(self, tensor_name, dtype, shape):
        """_create_shm_tensor (base.py:36-80): None for an empty shape; the existing segment
        while the tensor fits in it; else a new segment of 1.2x the size under a fresh name."""
        if isinstance(dtype, str):
            dtype = str2dtype(dtype)
        numel = 1
        for d in shape:
            numel *= int(d)
        if numel <= 0:
            return None
        need = numel * dtype_sizeof(dtype)
        old = self._shm_tensor_meta.get(tensor_name)
        if old is not None and need <= old.shm_size:
            self._shm_tensor_meta[tensor_name] = TensorMeta(old.shm_name, old.fd, old.ptr,
                                                            old.shm_size, dtype, shape)
            return open_shared_tensor(old.ptr, dtype, shape)
        if old is not None:
            release_shared_mem(old.shm_name, old.shm_size, old.ptr, old.fd, self._pin_memory)
            del self._shm_tensor_meta[tensor_name]
        size = int(need * SHM_ALLOC_AMPL_TIMES)
        shm_name = self._create_shm_name(tensor_name)
        ptr, fd = create_shared_mem(shm_name, size, self._pin_memory)
        self._shm_tensor_meta[tensor_name] = TensorMeta(shm_name, fd, ptr, size, dtype, shape)
        return open_shared_tensor(ptr, dtype, shape)

    def open(self, tensor_name, shm_name, shm_size, dtype, shape):
        """_open_shm_tensor (base.py:82-106): maps the peer's segment, dropping the mapping of an
        older segment of the same tensor."""
        old = self._shm_tensor_meta.get(tensor_name)
        if old is not None and old.shm_name == shm_name:
            self._shm_tensor_meta[tensor_name] = TensorMeta(shm_name, old.fd, old.ptr, shm_size,
                                                            dtype, shape)
            return open_shared_tensor(old.ptr, dtype, shape)
        if old is not None:
            release_shared_mem(old.shm_name, old.shm_size, old.ptr, old.fd, self._pin_memory)
            del self._shm_tensor_meta[tensor_name]
        ptr, fd = open_shared_mem(shm_name, shm_size, self._pin_memory)
        self._shm_tensor_meta[tensor_name] = TensorMeta(shm_name, fd, ptr, shm_size, dtype, shape)
        return open_shared_tensor(ptr, dtype, shape)

    def release(self, tensor_name):                                # base.py:108-111
        meta = self._shm_tensor_meta.pop(tensor_name)
        release_shared_mem(meta.shm_name, meta.shm_size, meta.ptr, meta.fd, self._pin_memory)

    def close(self):                                               # base.py:113-119
        for name in list(self._shm_tensor_meta):
            try:
                self.release(name)
            except RuntimeError:
                pass

    def __del__(self):
        self.close()
