"""The cache's bookkeeping lives in the kernel library as host code (csrc/host_cache.hip); this is
its binding.  Nothing here touches the GPU, so the library loads and works on a machine without one."""
from __future__ import annotations

from ctypes import POINTER, c_int, c_int32, c_long, c_void_p

from ..errors import CacheError

_lib = None

_SIGNATURES = {
    "ri_pool_new": ([c_int, c_int, c_int, c_int, c_int], c_void_p),
    "ri_pool_delete": ([c_void_p], None),
    "ri_pool_tables": ([c_void_p], POINTER(c_int32)),
    "ri_pool_free_count": ([c_void_p], c_int),
    "ri_pool_pages_needed": ([c_void_p, c_int, c_long, c_long], c_int),
    "ri_pool_reserve": ([c_void_p, c_int, c_long, c_long], c_int),
    "ri_pool_trim": ([c_void_p, c_int, c_long], c_int),
    "ri_pool_release": ([c_void_p, c_int], c_int),
    "ri_pool_check": ([c_void_p], c_int),
    "ri_cache_new": ([POINTER(c_void_p), c_int, c_int, c_int], c_void_p),
    "ri_cache_delete": ([c_void_p], None),
    "ri_cache_acquire": ([c_void_p], c_int),
    "ri_cache_release": ([c_void_p, c_int], c_int),
    "ri_cache_is_held": ([c_void_p, c_int], c_int),
    "ri_cache_check_held": ([c_void_p, c_int], c_int),
    "ri_cache_free_slots": ([c_void_p], c_int),
    "ri_cache_length": ([c_void_p, c_int], c_long),
    "ri_cache_longest": ([c_void_p, c_void_p, c_int], c_long),
    "ri_cache_reserve": ([c_void_p, c_void_p, c_void_p, c_int], c_int),
    "ri_cache_commit": ([c_void_p, c_void_p, c_void_p, c_int], c_int),
    "ri_cache_check": ([c_void_p], c_int),
    "ri_cache_plan_step": ([c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p,
                            c_long, c_void_p], c_long),
}


def lib():
    """The kernel library with the cache's functions typed."""
    global _lib
    if _lib is None:
        from ..kernels.build import load
        loaded = load()
        for name, (argtypes, restype) in _SIGNATURES.items():
            try:
                f = getattr(loaded, name)
            except AttributeError:
                raise CacheError(f"the kernel library has no {name}: it is older than this package, build it again") from None
            f.argtypes, f.restype = argtypes, restype
        _lib = loaded
    return _lib


def fail() -> CacheError:
    return CacheError(lib().ri_last_error().decode())


def check(rc: int) -> None:
    if rc != 0:
        raise fail()
