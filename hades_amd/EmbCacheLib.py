"""Drop-in for the reference's `EmbCacheLib` extension module on MI355X.

Same function names, argument names and argument order as the pybind module of the reference
(src/pybind.cc:46-70); the `cuda*` names are API names, not a CUDA dependency.  Each function
validates what the reference CHECKs (raising RuntimeError), allocates returned tensors with torch,
and calls the C-ABI library on torch's current stream.  Use it as

    import hades_amd.EmbCacheLib as EmbCacheLib
    # or, to serve `import EmbCacheLib` in unmodified reference code:
    import hades_amd; hades_amd.install_as_embcachelib()

Differences from the reference, all deliberate:
  * launches go to torch's current stream, not the legacy default stream;
  * HIP failures raise RuntimeError instead of exit() (src/utils.h:12-24);
  * tensors must be contiguous (the reference silently assumes it);
  * host tensors handed to a kernel must be page-locked.  cudaPin on a tensor that torch already
    pinned is a no-op; on pageable memory it tries hipHostRegister and raises if the platform
    refuses (allocate with `pinned_empty` / pin_memory=True instead).
"""
import ctypes

import torch

from . import _lib

_DTYPE = {torch.float32: _lib.F32, torch.float64: _lib.F64}
_ITYPE = {torch.int32: _lib.I32, torch.int64: _lib.I64}
_SPLIT_ITYPE = {torch.int64: _lib.I64, torch.int32: _lib.I32, torch.int16: _lib.I16,
                torch.int8: _lib.I8, torch.uint8: _lib.U8}

# storage pointers registered through cudaPin / cudaPinPtr by this module
_registered = set()


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """torch's current stream on the current device as a hipStream_t (the raw-handle query is an
    order of magnitude cheaper than building a torch.cuda.Stream object per call)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _dev(t, name):
    _check(t.is_cuda, "%s must be a device tensor" % name)
    _check(t.is_contiguous(), "%s must be contiguous" % name)


def _dev_or_pinned(t, name, contiguous=True):
    if contiguous:
        _check(t.is_contiguous(), "%s must be contiguous" % name)
    if not t.is_cuda:
        _check(t.is_pinned() or t.untyped_storage().data_ptr() in _registered,
               "%s is pageable host memory: pin it (cudaPin / pin_memory=True) before a kernel "
               "reads or writes it" % name)


def _dtype(t, name):
    _check(t.dtype in _DTYPE, "Type can only be float or double (%s is %s)" % (name, t.dtype))
    return _DTYPE[t.dtype]


def _itype(t, name):
    _check(t.dtype in _ITYPE, "ID can only be int32 or int64 (%s is %s)" % (name, t.dtype))
    return _ITYPE[t.dtype]


def _row_dim(ref, others):
    """dim of the row payload: 1 for 1-D tensors, size(1) for 2-D (src/cuda/uva_fetch.cu:73-81)."""
    _check(ref.dim() in (1, 2), "tensors must be 1-D or 2-D")
    for o in others:
        _check(o.dim() == ref.dim(), "tensors must have the same number of dimensions")
    if ref.dim() == 1:
        return 1
    for o in others:
        _check(o.size(1) == ref.size(1), "row widths differ")
    return ref.size(1)


def pinned_empty(shape, dtype=torch.float32):
    """A page-locked, device-mapped host tensor (what the cold table should live in)."""
    return torch.empty(shape, dtype=dtype, pin_memory=True)


_host_allocs = {}   # data_ptr -> (raw pointer, bytes) of tensors made by host_alloc


def host_alloc(shape, dtype=torch.float32, coherent=True):
    """A host tensor in memory from hades_host_alloc (page-locked and mapped into the device's
    address space: kernels read and write it zero-copy).  coherent=False asks for coarse-grained
    memory (see HADES_HOST_NONCOHERENT in the header).  Free it with host_free(tensor) once no
    kernel uses it any more; the tensor and its views must not be touched afterwards."""
    shape = tuple(int(x) for x in (shape if hasattr(shape, "__len__") else (shape,)))
    numel = 1
    for x in shape:
        numel *= x
    nbytes = numel * torch.empty((), dtype=dtype).element_size()
    if nbytes == 0:
        return torch.empty(shape, dtype=dtype)
    raw = ctypes.c_void_p()
    _lib.call("hades_host_alloc_flags", ctypes.byref(raw), nbytes,
              0 if coherent else _lib.HOST_NONCOHERENT)
    buf = (ctypes.c_char * nbytes).from_address(raw.value)
    t = torch.frombuffer(buf, dtype=dtype).view(shape)
    _host_allocs[t.data_ptr()] = (raw.value, nbytes)
    _registered.add(t.untyped_storage().data_ptr())
    return t


def host_free(tensor):
    """Gives the memory of a host_alloc tensor back (hades_host_free)."""
    ptr = tensor.data_ptr()
    _check(ptr in _host_allocs, "host_free: not a tensor made by host_alloc")
    raw, _ = _host_allocs.pop(ptr)
    _registered.discard(tensor.untyped_storage().data_ptr())
    _lib.call("hades_host_free", ctypes.c_void_p(raw))


# ---- pinning (src/cuda/pin_memory.cu:9-26) ----------------------------------
def cudaPin(tensor):
    if tensor.is_cuda or tensor.is_pinned():
        return
    ptr = tensor.untyped_storage().data_ptr()
    _lib.call("hades_pin", ctypes.c_void_p(ptr), tensor.numel() * tensor.element_size())
    _registered.add(ptr)


def cudaUnpin(tensor):
    ptr = tensor.untyped_storage().data_ptr()
    if ptr in _registered:
        _lib.call("hades_unpin", ctypes.c_void_p(ptr))
        _registered.discard(ptr)


def cudaPinPtr(ptr, size):
    _lib.call("hades_pin", ctypes.c_void_p(ptr), size)
    _registered.add(ptr)


def cudaUnpinPtr(ptr):
    _lib.call("hades_unpin", ctypes.c_void_p(ptr))
    _registered.discard(ptr)


# ---- split (src/cuda/split.cu:13-56) -----------------------------------------
def cudaSplit(ids, mask):
    _dev(ids, "ids")
    _dev_or_pinned(mask, "mask")
    _check(mask.dtype == torch.int8, "mask must be int8")
    _check(ids.dtype in _SPLIT_ITYPE, "ids must be an integer tensor (got %s)" % ids.dtype)
    n = ids.numel()
    out = torch.empty((3, n), dtype=torch.bool, device=ids.device)
    _lib.call("hades_split", _ptr(ids), _SPLIT_ITYPE[ids.dtype], _ptr(mask), n,
              _ptr(out[0]), _ptr(out[1]), _ptr(out[2]), _stream())
    return [out[0], out[1], out[2]]


# ---- gathers (src/cuda/uva_fetch.cu) -----------------------------------------
def cudaFetch(src, src_index, dst, dst_index):
    _dev_or_pinned(src, "src"); _dev(src_index, "src_index"); _dev(dst, "dst"); _dev(dst_index, "dst_index")
    _check(src.dim() == 2 and dst.dim() == 2, "cudaFetch takes 2-D tensors")
    _check(src.size(1) == dst.size(1), "src.size(1) == dst.size(1)")
    _check(dst_index.numel() == src_index.numel(), "dst_index.numel() == src_index.numel()")
    _check(src.dtype == dst.dtype and src_index.dtype == dst_index.dtype, "dtype mismatch")
    _lib.call("hades_fetch", _ptr(src), _ptr(src_index), _ptr(dst), _ptr(dst_index),
              src_index.numel(), src.size(1), _dtype(src, "src"), _itype(src_index, "src_index"),
              _stream())


def cudaFetch2(src, src_index, dst):
    _dev_or_pinned(src, "src"); _dev(src_index, "src_index"); _dev(dst, "dst")
    dim = _row_dim(src, [dst])
    _check(src.dtype == dst.dtype, "dtype mismatch")
    _check(dst.size(0) >= src_index.numel(), "dst has fewer rows than src_index has entries")
    _lib.call("hades_fetch2", _ptr(src), _ptr(src_index), _ptr(dst), src_index.numel(), dim,
              _dtype(src, "src"), _itype(src_index, "src_index"), _stream())


def cudaFetchWithCache2(cpu_src, gpu_src, src_index, index_map, dst):
    _dev_or_pinned(cpu_src, "cpu_src"); _dev(gpu_src, "gpu_src"); _dev(src_index, "src_index")
    _dev(index_map, "index_map"); _dev(dst, "dst")
    dim = _row_dim(gpu_src, [cpu_src, dst])
    _check(cpu_src.dtype == gpu_src.dtype == dst.dtype, "dtype mismatch")
    _check(index_map.dtype == src_index.dtype, "index_map and src_index must have the same dtype")
    _check(dst.size(0) >= src_index.numel(), "dst has fewer rows than src_index has entries")
    _lib.call("hades_fetch_with_cache2", _ptr(cpu_src), _ptr(gpu_src), _ptr(src_index),
              _ptr(index_map), _ptr(dst), src_index.numel(), dim, _dtype(gpu_src, "gpu_src"),
              _itype(src_index, "src_index"), _stream())


# ---- scatters (src/cuda/uva_set.cu, and the misnamed cudaCombine) -------------
def cudaSet(src, dst, dst_index):
    _dev(src, "src"); _dev_or_pinned(dst, "dst"); _dev(dst_index, "dst_index")
    dim = _row_dim(src, [dst])
    _check(src.dtype == dst.dtype, "dtype mismatch")
    _check(src.size(0) >= dst_index.numel(), "src has fewer rows than dst_index has entries")
    _lib.call("hades_set", _ptr(src), _ptr(dst), _ptr(dst_index), dst_index.numel(), dim,
              _dtype(src, "src"), _itype(dst_index, "dst_index"), _stream())


def cudaSetWithCache(src, cpu_dst, gpu_dst, dst_index, index_map):
    _dev(src, "src"); _dev_or_pinned(cpu_dst, "cpu_dst"); _dev(gpu_dst, "gpu_dst")
    _dev(dst_index, "dst_index"); _dev(index_map, "index_map")
    dim = _row_dim(src, [cpu_dst, gpu_dst])
    _check(src.dtype == cpu_dst.dtype == gpu_dst.dtype, "dtype mismatch")
    _check(index_map.dtype == dst_index.dtype, "index_map and dst_index must have the same dtype")
    _check(src.size(0) >= dst_index.numel(), "src has fewer rows than dst_index has entries")
    _lib.call("hades_set_with_cache", _ptr(src), _ptr(cpu_dst), _ptr(gpu_dst), _ptr(dst_index),
              _ptr(index_map), dst_index.numel(), dim, _dtype(src, "src"),
              _itype(dst_index, "dst_index"), _stream())


def cudaCombine(src, dst, dst_index):
    _dev(src, "src"); _dev_or_pinned(dst, "dst"); _dev(dst_index, "dst_index")
    _check(src.dim() == 2 and dst.dim() == 2, "cudaCombine takes 2-D tensors")
    _check(src.size(1) == dst.size(1), "src.size(1) == dst.size(1)")
    _check(src.dtype == dst.dtype, "dtype mismatch")
    _check(src.size(0) >= dst_index.numel(), "src has fewer rows than dst_index has entries")
    _lib.call("hades_combine_scatter", _ptr(src), _ptr(dst), _ptr(dst_index), dst_index.numel(),
              src.size(1), _dtype(src, "src"), _itype(dst_index, "dst_index"), _stream())


# ---- routing (src/cuda/binary_search.cu) --------------------------------------
def _first_arg(args, kwargs, name):
    if args:
        return args[0], args[1:]
    _check("in" in kwargs, "%s: missing argument 'in'" % name)
    return kwargs.pop("in"), args


def cudaReminder(*args, **kwargs):
    """cudaReminder(in, local_num_gpus) -> in % local_num_gpus"""
    in_, rest = _first_arg(args, kwargs, "cudaReminder")
    local_num_gpus = rest[0] if rest else kwargs.pop("local_num_gpus")
    _dev(in_, "in")
    out = torch.empty_like(in_)
    _lib.call("hades_reminder", _ptr(in_), int(local_num_gpus), _ptr(out), in_.size(0),
              _itype(in_, "in"), _stream())
    return out


def cudaBinarySearch(*args, **kwargs):
    """cudaBinarySearch(in, range_partition, local_num_gpus) -> owner rank of every id"""
    in_, rest = _first_arg(args, kwargs, "cudaBinarySearch")
    rest = list(rest)
    range_partition = rest.pop(0) if rest else kwargs.pop("range_partition")
    local_num_gpus = rest.pop(0) if rest else kwargs.pop("local_num_gpus")
    _dev(in_, "in"); _dev(range_partition, "range_partition")
    _check(range_partition.dtype == in_.dtype, "in and range_partition must have the same dtype")
    out = torch.empty_like(in_)
    _lib.call("hades_binary_search", _ptr(in_), _ptr(range_partition), range_partition.size(0),
              int(local_num_gpus), _ptr(out), in_.size(0), _itype(in_, "in"), _stream())
    return out


def cudaBinarySearch2(*args, **kwargs):
    """cudaBinarySearch2(in, range) -> number of entries of the ascending `range` that are <= in[i]"""
    in_, rest = _first_arg(args, kwargs, "cudaBinarySearch2")
    range_ = rest[0] if rest else kwargs.pop("range")
    _dev(in_, "in"); _dev(range_, "range")
    _check(range_.dtype == in_.dtype, "in and range must have the same dtype")
    out = torch.empty_like(in_)
    _lib.call("hades_binary_search2", _ptr(in_), _ptr(range_), range_.size(0), _ptr(out),
              in_.size(0), _itype(in_, "in"), _stream())
    return out


def __getattr__(name):
    """EmbCacheLib.IndexCache (src/pybind.cc:17-36), resolved on first use: the class lives in
    hades_amd.index_cache, which itself imports this module."""
    if name == "IndexCache":
        from .index_cache import IndexCache
        return IndexCache
    if name in ("create_shared_mem", "open_shared_mem", "release_shared_mem", "open_shared_tensor"):
        from . import shm                      # src/pybind.cc:38-45
        return getattr(shm, name)
    raise AttributeError("module %r has no attribute %r" % (__name__, name))
