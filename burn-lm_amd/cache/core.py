"""ctypes binding of the native host core (``csrc/host/cache_core.cpp``): the pool of pages, the
cache's bookkeeping and the assembly of a step's index arrays."""
from __future__ import annotations

import ctypes
import threading
from typing import List, Sequence

from ..csrc import build as _build

HOST_ABI = 4
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
    "blm_cache_advance_all": ([_ptr, _int, _ptr, _ptr], _int), "blm_cache_lengths": ([_ptr, _int, _ptr, _ints], _int),
    "blm_step_size": ([_int, _int, _int, _int, _int], _ll),
    # the five arrays of a step's entries come as addresses of array('i') buffers (see Packed)
    "blm_step_fill": ([_ptr, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _int, _int, _int, _ptr, _ll, _ints, _int], _int),
    "blm_step_check": ([_ptr, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _int], _int),
    "blm_step_key": ([_int, _ptr, _ints, _ptr, _ptr, _int, _ints, _int, _ints, _int, _int, _int, _ints], None),
    "blm_plan_batches": ([_int, _ints, _int, _int, _int, _int, _int, _int, _ints], _int),
    "blm_plan_prompt_steps": ([_int, _ints, _int, _int, _ints, _ints, _ints, _ints], _int),
    "blm_gen_new": ([_int, _ints, _int, _int, _int, _ints], _ptr), "blm_gen_free": ([_ptr], None),
    "blm_gen_start": ([_ptr, _int, _ints], _int), "blm_gen_ahead_rows": ([_ptr, _ints], _int),
    "blm_gen_launched": ([_ptr, _int, _ints], _int), "blm_gen_take": ([_ptr, _ints, _ints], _int),
    "blm_gen_live": ([_ptr, _ints, _ints], _int), "blm_gen_count": ([_ptr, _int], _int),
    "blm_uniforms": ([ctypes.c_ulonglong, _int, _ints, _ints, _ptr], None),
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


class Packed:
    """The entries of one step, (slot, tokens, wanted places) per sequence, as five flat int32 arrays
    that the native core reads in place: slots, token counts, all tokens, want counts, all wanted
    places.  Built at C speed; anything that is no integer (a float, a string) raises TypeError, an
    integer that does not fit 32 bits OverflowError."""
    __slots__ = ("n", "slots", "counts", "tokens", "want_counts", "wants", "_keep")

    def __init__(self, entries):
        from array import array
        slots, counts, tokens, want_counts, wants = array("i"), array("i"), array("i"), array("i"), array("i")
        for slot, toks, want in entries:
            slots.append(slot)
            counts.append(len(toks))
            tokens.extend(toks)
            want_counts.append(len(want))
            wants.extend(want)
        for a in (tokens, wants):       # an address of an empty array is not one the core may read: give it a word
            if not len(a):
                a.append(0)
        self.n = len(slots)
        self._keep = (slots, counts, tokens, want_counts, wants)
        self.slots, self.counts, self.tokens, self.want_counts, self.wants = (a.buffer_info()[0] for a in self._keep)

    @classmethod
    def one_token_each(cls, slots):
        """A decode step's entries whose tokens are not known to the host: token 0, its place wanted."""
        from array import array
        n = len(slots)
        self = cls.__new__(cls)
        self.n = n
        self._keep = (array("i", slots), array("i", [1]) * n, array("i", [0]) * n, array("i", [1]) * n, array("i", [0]) * n)
        self.slots, self.counts, self.tokens, self.want_counts, self.wants = (a.buffer_info()[0] for a in self._keep)
        return self

    def slot_list(self):
        return self._keep[0].tolist()

    def count_list(self):
        return self._keep[1].tolist()

    @property
    def n_tokens(self):
        return sum(self._keep[1])

    @property
    def n_wanted(self):
        return sum(self._keep[3])


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
