"""hades_amd - the HADES per-GPU embedding-cache hot path on MI355X (gfx950).

    hades_amd.EmbCacheLib   drop-in for the reference's extension module (same operator names)
    hades_amd.ops           fused operators: lookup, split, cached_fetch/set, combine, optimizers
    hades_amd.cache         EmbCache: hot-row cache keyed by the sorted hot-ID set
    hades_amd.sparse_optim  only_unique_grads / unique_grads / bucket_gradients / SparseAdagrad / SparseAdam
    hades_amd.dist_emb      DistEmb / DistEmbeddingTensor and the trace-driven SparseAdam / SparseAdagrad
    hades_amd.index_cache   IndexCache / LocalCache: the set-associative index cache, in HBM
    hades_amd.cold_cache    ColdDataCache: the cache server's gradient path with its staleness rule
    hades_amd.shm           shared-memory segments and tensors, ShmTensorPool

All device work is done by csrc/libhades_hip.so (hand-written HIP, C ABI in include/hades_hip.h),
built in-tree with `python -m hades_amd.build`.  There is no CPU fallback: without the library
every operator raises.
"""
import sys

__version__ = "0.1.0"


def install_as_embcachelib():
    """Registers hades_amd.EmbCacheLib under the name `EmbCacheLib`, so that unmodified reference
    code (`import EmbCacheLib`, python/EmbCache/cache.py:2) binds to this implementation.

    What differs from the reference's module for such code: launches go to torch's current stream;
    failures raise RuntimeError instead of ending the process; tensors must be contiguous; host
    tensors given to a kernel must be page-locked already (cudaPin on pageable memory raises where
    the platform refuses hipHostRegister: allocate with pin_memory=True or EmbCacheLib.host_alloc);
    IndexCache lives in device memory, ignores its shared-memory arguments, accepts CPU or device
    id tensors (CPU in, CPU out) and returns device tensors from getall."""
    from . import EmbCacheLib
    sys.modules["EmbCacheLib"] = EmbCacheLib
    return EmbCacheLib
