"""ctypes binding of the native host core (``csrc/host/cache_core.cpp``): the pool of pages, the
cache's bookkeeping and the assembly of a step's index arrays."""
from __future__ import annotations

import ctypes
import threading
from typing import List, Sequence

from ..csrc import build as _build

HOST_ABI = 2
OK, E_FULL, E_OVERFLOW, E_USAGE = 0, 1, 2, 3

_lib = None
_lock = threading.Lock()
_int, _ptr, _ll = ctypes.c_int, ctypes.c_void_p, ctypes.c_longlong
_ints = ctypes.POINTER(ctypes.c_int)

_SIGNATURES = {
    "blm_pool_new": ([_int], _ptr), "blm_pool_free": ([_ptr], None), "blm_pool_n_free": ([_ptr], _int),
    "blm_pool_take": ([_ptr, _int, _ints], _int), "blm_pool_give": ([_ptr, _int, _ints], _int),
    "blm_pool_free_list": ([_ptr, _ints], _int), "blm_pool_is_out": ([_ptr, _int], _int),
    "blm_cache_new": ([_int, _ints, _ints, _int, _int, _int], _ptr), "blm_cache_free": ([_ptr], None),
    "blm_cache_open": ([_ptr, _ints], _int), "blm_cache_close": ([_ptr, _int], _int),
    "blm_cache_length": ([_ptr, _int], _int), "blm_cache_reserve": ([_ptr, _int, _ints, _ints, _ints], _int),
    "blm_cache_advance": ([_ptr, _int, _int], _int), "blm_cache_table_len": ([_ptr, _int, _int], _int),
    "blm_cache_table": ([_ptr, _int, _int, _ints], _int),
    "blm_cache_page_table": ([_ptr, _int, _int, _ints, _int, _ints], _int), "blm_cache_pool": ([_ptr, _int], _ptr),
    "blm_cache_n_free_slots": ([_ptr], _int), "blm_cache_free_slots": ([_ptr, _ints], _int),
    "blm_cache_live_slots": ([_ptr, _ints], _int),
    "blm_step_size": ([_int, _int, _int, _int, _int], _ll),
    "blm_step_fill": ([_ptr, _int, _ints, _ints, _ints, _ints, _ints, _int, _int, _int, _ptr, _ll, _ints], _int),
}


def library():
    """The loaded host library; compiled at the first call if it is not there."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                path = _build.ensure_host_built()
                lib = ctypes.CDLL(path)
                lib.blm_host_abi_version.restype = _int
                if lib.blm_host_abi_version() != HOST_ABI:
                    raise RuntimeError(f"{path} has ABI {lib.blm_host_abi_version()}, expected {HOST_ABI}: rebuild it")
                lib.blm_host_last_error.restype = ctypes.c_char_p
                for name, (args, res) in _SIGNATURES.items():
                    fn = getattr(lib, name)
                    fn.argtypes, fn.restype = args, res
                _lib = lib
    return _lib


def last_error() -> str:
    return library().blm_host_last_error().decode()


def ints(values: Sequence[int]):
    return (ctypes.c_int * len(values))(*values)


class NativePool:
    """A pool of page numbers: either its own object or a view of one group's pool inside a cache."""

    def __init__(self, n_pages: int, handle=None):
        self._lib = library()
        self.n_pages = n_pages
        self._own = handle is None     # a view (handle given) is valid only as long as its cache
        self._h = self._lib.blm_pool_new(n_pages) if handle is None else handle
        if not self._h:
            raise ValueError(f"bad pool size {n_pages}")

    def __del__(self):
        if getattr(self, "_own", False) and self._h:
            self._lib.blm_pool_free(self._h)
            self._h = None

    @property
    def n_free(self) -> int:
        return self._lib.blm_pool_n_free(self._h)

    def take(self, n: int):
        out = (ctypes.c_int * max(n, 1))()
        return self._lib.blm_pool_take(self._h, n, out), list(out[:n])

    def give(self, pages: Sequence[int]) -> int:
        return self._lib.blm_pool_give(self._h, len(pages), ints(list(pages)))

    def free_list(self) -> List[int]:
        out = (ctypes.c_int * max(self.n_pages, 1))()
        n = self._lib.blm_pool_free_list(self._h, out)
        return list(out[:n])

    def out_set(self):
        return {p for p in range(self.n_pages) if self._lib.blm_pool_is_out(self._h, p)}
