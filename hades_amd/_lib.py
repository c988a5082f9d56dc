"""ctypes binding of libhades_hip.so (declared in include/hades_hip.h).

The library is the product: there is no fallback.  If it has not been built, loading raises
with the build command; if a call fails, the library's own message is raised as RuntimeError
(the reference's CHECK(...) failures surface in Python as RuntimeError too: src/cuda/uva_fetch.cu:30-31).
"""
import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
# HADES_LIB_PATH selects another build of the same library (e.g. one compiled with other tuning
# constants); by default the in-tree build is used.
LIB_PATH = os.environ.get("HADES_LIB_PATH") or os.path.join(_HERE, "csrc", "libhades_hip.so")

F32, F64 = 0, 1
I32, I64, I16, I8, U8 = 0, 1, 2, 3, 4
COMBINE_FAST, COMBINE_EXACT = 0, 1
HOST_NONCOHERENT = 1
COMBINE_STATIC_SCRATCH_BYTES = 16 << 20

_P = c_void_p
_L = c_int64

# name -> argument types; every function returns int unless listed in _RESTYPE
KERNEL_NONE, KERNEL_CACHED_FETCH, KERNEL_SEG_SUM, KERNEL_ADAGRAD, KERNEL_RADIX_PASS = 0, 1, 2, 3, 4
KERNEL_HASH_ACCUMULATE = 5
KERNEL_ADAM = 6
ABI_VERSION = 131      # HADES_ABI_VERSION of include/hades_hip.h

_SIGNATURES = {
    "hades_profile_kernel": [c_int, _P, _P],
    "hades_set_host_link_blocks": [c_int, _L],
    "hades_sort_config": [c_int, _L],
    "hades_pin": [_P, c_size_t],
    "hades_unpin": [_P],
    "hades_host_alloc": [ctypes.POINTER(c_void_p), c_size_t],
    "hades_host_alloc_flags": [ctypes.POINTER(c_void_p), c_size_t, ctypes.c_uint],
    "hades_host_free": [_P],
    "hades_shm_create": [c_char_p, _L, c_int, ctypes.POINTER(c_void_p), ctypes.POINTER(c_int64)],
    "hades_shm_open": [c_char_p, _L, c_int, ctypes.POINTER(c_void_p), ctypes.POINTER(c_int64)],
    "hades_shm_release": [c_char_p, _L, _P, _L, c_int],
    "hades_shm_exists": [c_char_p],
    "hades_fetch": [_P, _P, _P, _P, _L, _L, c_int, c_int, _P],
    "hades_fetch2": [_P, _P, _P, _L, _L, c_int, c_int, _P],
    "hades_fetch_with_cache2": [_P, _P, _P, _P, _P, _L, _L, c_int, c_int, _P],
    "hades_set": [_P, _P, _P, _L, _L, c_int, c_int, _P],
    "hades_set_with_cache": [_P, _P, _P, _P, _P, _L, _L, c_int, c_int, _P],
    "hades_combine_scatter": [_P, _P, _P, _L, _L, c_int, c_int, _P],
    "hades_reminder": [_P, _L, _P, _L, c_int, _P],
    "hades_binary_search": [_P, _P, _L, _L, _P, _L, c_int, _P],
    "hades_binary_search2": [_P, _P, _L, _P, _L, c_int, _P],
    "hades_split": [_P, c_int, _P, _L, _P, _P, _P, _P],
    "hades_lookup_sorted": [_P, _L, _P, _L, _P, _P, _P],
    "hades_hot_index_build": [_P, _L, _P, c_size_t, _P],
    "hades_split_compact": [_P, _L, _P, _P, _P, _P, _P, c_size_t, _P],
    "hades_split3_compact": [_P, c_int, _P, _L, _P, _P, _P, _P, _P, _P, _P, _P, c_size_t, _P],
    "hades_lookup_split": [_P, _P, _L, _P, _L, _P, _P, _P, _P, _P, _P, _P, c_int, _P, c_size_t, _P],
    "hades_fetch_listed": [_P, _L, _P, _P, _P, _L, _P, _L, c_int, _P],
    "hades_fetch_listed_in_set": [_P, _L, _P, _P, _P, _L, _P, _P, _L, _P, _L, c_int, _P],
    "hades_set_listed": [_P, _P, _L, _P, _P, _P, _L, _L, c_int, _P],
    "hades_adagrad_update_listed": [_P, _P, _P, _P, _L, _L, _P, _P, _L, _P, c_float, c_float, _P],
    "hades_cached_fetch": [_P, _P, _P, _L, _P, _L, _P, _P, _P, _L, c_int, _P],
    "hades_cached_fetch_loc": [_P, _P, _P, _P, _L, _P, _L, c_int, _P],
    "hades_cached_set": [_P, _P, _P, _P, _L, _P, _L, _P, _L, c_int, _P],
    "hades_combine": [_P, _P, _L, _L, _L, c_int, _P, _P, _P, _P, _P, _P, c_size_t, _P],
    "hades_combine_plan_classed": [_P, _L, _L, _L, _L, _P, _P, _P, _P, _P, c_size_t, _P],
    "hades_combine_apply_class": [_P, _L, _L, _L, c_int, c_int, _P, _P, _P, _P, _P, c_size_t, _P],
    "hades_adagrad_update_class": [_P, _P, _P, _P, c_int, _L, _L, _L, _P, _P, _L, _P, _P, _P, c_int,
                                   c_float, c_float, _P],
    "hades_adagrad_update_class_summing": [_P, _P, _L, _L, _P, _P, c_int, _L, _L, _P, _P, _L, _P, _P, _P, _P,
                                           c_int, c_float, c_float, _P, c_size_t, _P],
    "hades_adam_update_class_summing": [_P, _P, _L, _L, _P, _P, c_int, _L, _L, _P, _P, _P, _P, _L, _P, _P,
                                        _P, _P, c_int, c_float, ctypes.c_double, ctypes.c_double, c_float, _P,
                                        c_size_t, _P],
    "hades_combine_static": [_P, _P, _L, _L, _L, c_int, _P, _P, _P, _P, _P, _P],
    "hades_combine_plan": [_P, _L, _L, _L, _P, _P, _P, _P, c_size_t, _P],
    "hades_combine_apply": [_P, _L, _L, _L, c_int, _P, _P, _P, _P, c_size_t, _P],
    "hades_rows_div_count": [_P, _P, _P, _L, _L, c_int, _P],
    "hades_adagrad_update": [_P, _P, _P, _L, _L, _P, _L, _P, _P, _P, _P, _P, _P, c_int, c_float, c_float, _P],
    "hades_adam_update": [_P, _P, _P, _L, _L, _P, _L, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_int,
                          c_float, ctypes.c_double, ctypes.c_double, c_float, _P],
    "hades_adam_update_listed": [_P, _P, _P, _P, _L, _L, _P, _P, _P, _P, _L, c_float,
                                 ctypes.c_double, ctypes.c_double, c_float, _P],
    "hades_adam_update_class": [_P, _P, _P, _P, c_int, _L, _L, _L, _P, _P, _P, _P, _L, _P, _P, _P, c_int,
                                c_float, ctypes.c_double, ctypes.c_double, c_float, _P],
    "hades_hash_clear": [_P, _P, _P, _L, _L, _L, _P],
    "hades_hash_accumulate": [_P, _P, _P, _L, _P, _P, _P, _P, _L, _L, _P, _L, _P],
    "hades_hash_flush": [_P, _P, _P, _L, _L, _L, _P, _P, _P, _P, _L, _P, _L, _P, c_size_t, _P],
    "hades_bucket_by_owner": [_P, _L, _P, _L, _L, _L, _P, _L, c_int, _P, _P, _P, _P, _P, _P, _P,
                              c_size_t, _P],
    "hades_sacache_init": [_P, _P, _L, _P],
    "hades_sacache_add": [_P, _P, _L, _P, _L, _P, _P, c_size_t, _P],
    "hades_sacache_lookup": [_P, _L, _P, _L, _P, _P],
    "hades_sacache_lookup_touch": [_P, _P, _L, _P, _L, _P, _P, c_size_t, _P],
    "hades_sacache_reset": [_P, _P, _L, _P, _L, _P],
    "hades_sacache_getall": [_P, _L, _P, _P, _P, _P, _L, _P, c_size_t, _P],
    "hades_coldcache_insert": [_P, _P, _P, _P, _L, _L, _L, _P, _P, _P, _P, _P],
    "hades_coldcache_accumulate": [_P, _P, _P, _L, _L, _L, _L, _P, _P, _P, _P, _P, _P],
    "hades_coldcache_flush": [_L, _L, c_int, _L, _P, _P, _P, _P, _P, _P, _P, _L, _P, _P, _P, _P,
                              _L, _P, c_size_t, _P],
}
_SIZE_QUERIES = {
    "hades_sort_mode": [],
    "hades_get_host_link_blocks": [c_int],
    "hades_split_compact_workspace_bytes": [_L],
    "hades_hot_index_bytes": [_L],
    "hades_combine_workspace_bytes": [_L, _L],
    "hades_combine_workspace_bytes_min": [_L, _L],
    "hades_hash_flush_workspace_bytes": [_L, _L],
    "hades_bucket_workspace_bytes": [_L],
    "hades_sacache_workspace_bytes": [_L],
    "hades_sacache_getall_workspace_bytes": [_L],
    "hades_coldcache_flush_workspace_bytes": [_L],
}

_lib = None


def load():
    """Returns the loaded library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "%s is missing: build it with `python -m hades_amd.build` (needs hipcc). "
            "There is no CPU fallback." % LIB_PATH)
    # torch wheels bundle their own HIP runtime (same soname as the system one).  It has to be in
    # the process before this library is opened, so that both bind to ONE runtime and torch's
    # streams and allocations mean something to these kernels; the other order gives two runtimes.
    import torch  # noqa: F401
    lib = ctypes.CDLL(LIB_PATH)
    lib.hades_last_error.restype = c_char_p
    lib.hades_last_error.argtypes = []
    lib.hades_version.restype = c_int
    lib.hades_version.argtypes = []
    if lib.hades_version() != ABI_VERSION:
        raise RuntimeError("%s was built from other sources (interface version %d, this binding "
                           "expects %d): rebuild it with `python -m hades_amd.build`"
                           % (LIB_PATH, lib.hades_version(), ABI_VERSION))
    for name, argtypes in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = c_int
        fn.argtypes = argtypes
    for name, argtypes in _SIZE_QUERIES.items():
        fn = getattr(lib, name)
        fn.restype = c_size_t
        fn.argtypes = argtypes
    _lib = lib
    return lib


def exported_names():
    return ["hades_last_error", "hades_version"] + list(_SIGNATURES) + list(_SIZE_QUERIES)


def call(name, *args):
    """Calls an int-returning entry point and raises RuntimeError with the library's message."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        msg = lib.hades_last_error().decode("utf-8", "replace")
        raise RuntimeError("%s failed (code %d): %s" % (name, rc, msg))


def query(name, *args):
    return int(getattr(load(), name)(*args))
