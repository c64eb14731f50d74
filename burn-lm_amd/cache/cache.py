"""The cache: what every live sequence holds between steps.

A *slot* belongs to one sequence from ``open()`` to ``close()``.  For every place in the layer
order that keeps keys and values, a sequence owns pages of ``page_size`` tokens, handed out from
a pool as the sequence grows and given back when it ends; each sequence has its own length.
Places with the same need (key-value heads, head size, window) form a *group* that shares one
storage tensor, one pool and one page table, so layers that keep all keys and layers that keep
a window never compete for the same pages.  Beside the pages a sequence owns one row of each
fixed-size state tensor, zeroed when the slot is opened.

The reference keeps ``[max_batch, kv_heads, max_seq_len, head_dim]`` per layer with a single
length for the whole batch (crates/burn-lm-llama/src/nn/attention/cache.rs:19-35,
kv_cache.rs:14-33) and never clears it on reset (cache.rs:45-48); neither does this cache:
what a sequence may read is decided by its length alone, never by the bytes left in a page.

All bookkeeping is on the host and needs no GPU; only the storage tensors live on the device.
It is kept by the native core (csrc/host/cache_core.cpp, bound in core.py): slots, lengths, pools
and page tables, and the assembly of a step's index arrays; this module owns the tensors and
turns the core's failure codes into exceptions.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..parts.base import KVNeed, StateNeed
from . import core as _core


class CacheError(RuntimeError):
    pass


class CacheFull(CacheError):
    """No slot or not enough pages are free; nothing was changed."""


class ContextOverflow(CacheError):
    """A sequence would grow past the longest context the cache was built for; nothing was changed."""

    def __init__(self, actual, maximum):
        super().__init__(f"context length exceeded: {actual} tokens, maximum {maximum}")
        self.actual, self.maximum = actual, maximum


def _raise(code: int):
    """Turns a failure code of the native core into this module's exceptions."""
    msg = _core.last_error()
    if code == _core.E_FULL:
        raise CacheFull(msg)
    raise CacheError(msg)


class PagePool:
    """Free list of page numbers that knows which pages are out, so a page cannot be handed out
    twice or given back twice.  The list lives in the native core; a group's pool is a view of
    the one inside the cache's core."""

    def __init__(self, n_pages: int, _native=None):
        self.n_pages = n_pages
        self._native = _native if _native is not None else _core.NativePool(n_pages)

    @property
    def n_free(self):
        return self._native.n_free

    def take(self, n: int) -> List[int]:
        code, pages = self._native.take(n)
        if code:
            _raise(code)
        return pages

    def give(self, pages: Sequence[int]) -> None:
        code = self._native.give(pages)
        if code:
            _raise(code)

    # what tests look at: the free pages (the next to be handed out last) and the pages that are out
    @property
    def _free(self):
        return self._native.free_list()

    @property
    def _out(self):
        return self._native.out_set()


class _Tables:
    """Read-only mapping slot -> pages of each page index (-1 once released) of one group."""

    def __init__(self, cache, group_index):
        self._cache, self._gi = cache, group_index

    def __getitem__(self, slot):
        return self._cache._table(self._gi, slot)

    def __contains__(self, slot):
        return slot in self._cache.live_slots

    def __iter__(self):
        return iter(self._cache.live_slots)

    def __len__(self):
        return len(self._cache.live_slots)

    def keys(self):
        return self._cache.live_slots

    def values(self):
        return [self[s] for s in self._cache.live_slots]

    def items(self):
        return [(s, self[s]) for s in self._cache.live_slots]


class KVGroup:
    def __init__(self, need: KVNeed, places: List[Tuple], n_pages: int, page_size: int, dtype, device):
        # places: (place of the layer order, index among that place's needs or None if it has one) per plane
        self.need, self.places = need, places
        self.page_size = page_size
        self.n_pages = n_pages
        # keys [place in group, page, kv head, token in page * head_dim]: a key page is [token][head_dim];
        # values [place in group, page, value head, value_dim * token in page]: a value page is stored
        # transposed, [value_dim][token].  Keys and values have storage of their own, so their head sizes
        # and counts may differ.
        self.k_storage = torch.empty(len(places), n_pages, need.n_kv_heads, page_size * need.head_dim,
                                     dtype=dtype, device=device)
        self.v_storage = torch.empty(len(places), n_pages, need.v_heads, need.v_dim * page_size,
                                     dtype=dtype, device=device)
        self.pool: Optional[PagePool] = None      # set by the cache once its core exists
        self.tables: Optional[_Tables] = None

    def pages_for(self, length: int) -> int:
        return (length + self.page_size - 1) // self.page_size

    def first_needed_page(self, length_after: int) -> int:
        """Pages wholly before the window of the *next* query are never read again."""
        if self.need.window <= 0:
            return 0
        first_key = max(0, length_after - self.need.window + 1)  # oldest key the next token may see
        return first_key // self.page_size


class KVView:
    """What an attention-like mixer gets for its place in the order: the two storage planes, the
    page geometry, and (per step) the page table of the step's sequences."""

    def __init__(self, group: KVGroup, group_index: int, plane: int, store: bool):
        self.group_index, self.store = group_index, store
        n_pages, need = group.k_storage.shape[1], group.need
        self.k = group.k_storage[plane].view(n_pages, need.n_kv_heads, group.page_size, need.head_dim)
        self.v = group.v_storage[plane].view(n_pages, need.v_heads, need.v_dim, group.page_size)
        self.page_size = group.page_size
        self.need = group.need

    def block_table(self, step):
        return step.block_tables[self.group_index]


class StateView:
    """Fixed-size state of every slot for one place in the order: ``tensor[slot]``."""

    def __init__(self, tensor):
        self.tensor = tensor
        self.store = True


class Cache:
    """needs[i] is what place i of the layer order keeps: a KVNeed, a StateNeed, None, or a tuple
    of them for a block whose parts each keep something of their own (keys and values beside a
    state, two sets of keys and values); its view is then a tuple in the same order.
    reads_from[i] is the earlier place whose keys and values place i reads instead of keeping
    its own (or None); both places then have one need each."""

    def __init__(self, needs: Sequence, reads_from: Sequence[Optional[int]], max_tokens: int,
                 max_seqs: int, max_context: int, page_size: int = 64, dtype=torch.bfloat16,
                 device="cpu"):
        if max_tokens <= 0 or max_seqs <= 0 or max_context <= 0 or page_size <= 0:
            raise CacheError("cache sizes must be positive")
        self.page_size = page_size
        self.max_context = max_context
        self.max_seqs = max_seqs
        self.n_pages = (max_tokens + page_size - 1) // page_size
        self.table_width = (max_context + page_size - 1) // page_size
        self.groups: List[KVGroup] = []
        self.state_tensors: List[torch.Tensor] = []
        # a cell is one need: (place, None) for a place with one need, (place, j) for the j-th of several
        cells: List[Tuple] = []
        for i, need in enumerate(needs):
            if isinstance(need, (tuple, list)):
                if reads_from[i] is not None:
                    raise CacheError(f"place {i} of the layer order has several needs and keeps them all itself: "
                                     f"it cannot read the cache of place {reads_from[i]}")
                cells += [((i, j), n) for j, n in enumerate(need)]
            else:
                cells.append(((i, None), need))
        for key, need in cells:
            if need is not None and not isinstance(need, (KVNeed, StateNeed)):
                raise CacheError(f"place {key[0]} of the layer order asks for {need!r}: a need is a KVNeed, a StateNeed, "
                                 f"None or a tuple of them")
        cell_views: Dict[Tuple, object] = {key: None for key, _ in cells}
        by_need: Dict[KVNeed, List[Tuple]] = {}
        for key, need in cells:
            if reads_from[key[0]] is None and isinstance(need, KVNeed):
                by_need.setdefault(need, []).append(key)
        for need, keys in by_need.items():
            g = KVGroup(need, keys, self.n_pages, page_size, dtype, device)
            gi = len(self.groups)
            self.groups.append(g)
            for plane, key in enumerate(keys):
                cell_views[key] = KVView(g, gi, plane, store=True)
        for key, need in cells:
            i = key[0]
            src = reads_from[i]
            if src is not None:
                sv = cell_views.get((src, None)) if 0 <= src < i else None
                if reads_from[src] is not None or not isinstance(sv, KVView):
                    raise CacheError(f"place {i} of the layer order reads the cache of place {src}, which must be "
                                     f"an earlier place that keeps keys and values of its own")
                if isinstance(need, KVNeed) and (need.n_kv_heads, need.head_dim, need.v_heads, need.v_dim) != \
                        (sv.need.n_kv_heads, sv.need.head_dim, sv.need.v_heads, sv.need.v_dim):
                    raise CacheError(f"place {i} cannot read the cache of place {src}: head counts or sizes differ")
                g = self.groups[sv.group_index]
                cell_views[key] = KVView(g, sv.group_index, g.places.index((src, None)), store=False)
            elif isinstance(need, StateNeed):
                t = torch.zeros(max_seqs, *need.shape, dtype=need.dtype, device=device)
                self.state_tensors.append(t)
                cell_views[key] = StateView(t)
        self.views: List = []
        for i, need in enumerate(needs):
            if isinstance(need, (tuple, list)):
                self.views.append(tuple(cell_views[(i, j)] for j in range(len(need))))
            else:
                self.views.append(cell_views[(i, None)])
        lib = _core.library()
        self._lib = lib
        self._h = lib.blm_cache_new(len(self.groups), _core.ints([g.n_pages for g in self.groups]),
                                    _core.ints([g.need.window for g in self.groups]), page_size, max_seqs, max_context)
        if not self._h:
            raise CacheError("the native cache core refused these sizes")
        for gi, g in enumerate(self.groups):
            g.pool = PagePool(g.n_pages, _native=_core.NativePool(g.n_pages, handle=lib.blm_cache_pool(self._h, gi)))
            g.tables = _Tables(self, gi)

    def bytes_read(self, length: int) -> int:
        """Bytes of keys and values that one step reads for a sequence of `length` tokens: every
        place of the order reads its group's keys and values (a place that shares another's cache
        reads them again), all of them or the last window."""
        total = 0
        for v in (c for v in self.views for c in (v if isinstance(v, tuple) else (v,))):
            if isinstance(v, KVView):
                keys = min(length, v.need.window) if v.need.window > 0 else length
                total += (v.need.n_kv_heads * v.need.head_dim + v.need.v_heads * v.need.v_dim) * keys * v.k.element_size()
        return total

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.blm_cache_free(h)

    # ---- slots -----------------------------------------------------------------------------
    @property
    def free_slots(self):
        return self._lib.blm_cache_n_free_slots(self._h)

    @property
    def _free_slots(self):
        out = (_core.ctypes.c_int * self.max_seqs)()
        n = self._lib.blm_cache_free_slots(self._h, out)
        return list(out[:n])

    @property
    def live_slots(self):
        out = (_core.ctypes.c_int * self.max_seqs)()
        n = self._lib.blm_cache_live_slots(self._h, out)
        return list(out[:n])

    def open(self) -> int:
        slot = _core.ctypes.c_int(-1)
        code = self._lib.blm_cache_open(self._h, _core.ctypes.byref(slot))
        if code:
            _raise(code)
        for t in self.state_tensors:
            t[slot.value].zero_()
        return slot.value

    def close(self, slot: int) -> None:
        code = self._lib.blm_cache_close(self._h, int(slot))
        if code:
            _raise(code)

    def length(self, slot: int) -> int:
        n = self._lib.blm_cache_length(self._h, int(slot))
        if n < 0:
            raise CacheError(f"slot {slot} is not open")
        return n

    def room(self, slot: int) -> int:
        return self.max_context - self.length(slot)

    def _table(self, group_index: int, slot: int) -> List[int]:
        n = self._lib.blm_cache_table_len(self._h, group_index, int(slot))
        if n < 0:
            raise KeyError(slot)
        out = (_core.ctypes.c_int * max(n, 1))()
        self._lib.blm_cache_table(self._h, group_index, int(slot), out)
        return list(out[:n])

    # ---- growth ----------------------------------------------------------------------------
    def reserve(self, growth: Sequence) -> None:
        """growth: (slot, n_new) pairs of one step.  Hands out the pages all of them need, or
        raises before anything changed."""
        growth = list(growth)
        detail = (_core.ctypes.c_int * 2)()
        code = self._lib.blm_cache_reserve(self._h, len(growth), _core.ints([int(s) for s, _ in growth]),
                                           _core.ints([int(n) for _, n in growth]), detail)
        if code == _core.E_OVERFLOW:
            raise ContextOverflow(detail[0], detail[1])
        if code:
            _raise(code)

    def advance(self, slot: int, n: int) -> None:
        """The step that reserved n tokens for the slot has run: the sequence is n longer."""
        code = self._lib.blm_cache_advance(self._h, int(slot), int(n))
        if code:
            _raise(code)

    def page_table(self, group_index: int, slots: Sequence[int], width: int) -> List[List[int]]:
        slots = [int(s) for s in slots]
        out = (_core.ctypes.c_int * max(len(slots) * width, 1))()
        code = self._lib.blm_cache_page_table(self._h, group_index, len(slots), _core.ints(slots), width, out)
        if code:
            _raise(code)
        return [list(out[i * width:(i + 1) * width]) for i in range(len(slots))]

    # ---- a step's entries, packed (cache.core.Packed) ------------------------------------------
    def check_step(self, packed, vocab: int) -> None:
        """Slots open, at least one token each, tokens inside the vocabulary, wanted places inside each
        sequence's tokens: CacheError with the first fault's text, nothing changed."""
        code = self._lib.blm_step_check(self._h, packed.n, packed.slots, packed.counts, packed.tokens,
                                        packed.want_counts, packed.wants, int(vocab))
        if code:
            _raise(code)

    def reserve_step(self, packed) -> None:
        detail = (_core.ctypes.c_int * 2)()
        code = self._lib.blm_cache_reserve(self._h, packed.n, _core.ctypes.cast(packed.slots, _core._ints),
                                           _core.ctypes.cast(packed.counts, _core._ints), detail)
        if code == _core.E_OVERFLOW:
            raise ContextOverflow(detail[0], detail[1])
        if code:
            _raise(code)

    def advance_step(self, packed) -> None:
        code = self._lib.blm_cache_advance_all(self._h, packed.n, packed.slots, packed.counts)
        if code:
            _raise(code)

    def lengths_of(self, packed):
        out = (_core.ctypes.c_int * max(packed.n, 1))()
        code = self._lib.blm_cache_lengths(self._h, packed.n, packed.slots, out)
        if code:
            _raise(code)
        return out

    def fill_step(self, entries, pad_seqs: int, pad_tokens: int, width: int, out_ptr: int, capacity: int, vocab: int = 0):
        """Writes the index arrays of a step for entries ((slot, tokens, want) tuples, or a Packed) into
        int32 host memory at out_ptr (see blm_step_fill in csrc/host/cache_core.h for the layout and for
        the padding to pad_seqs sequences and pad_tokens tokens; 0: none) and returns (tokens, wanted
        rows, most tokens of one sequence, greatest length after the step)."""
        packed = entries if isinstance(entries, _core.Packed) else _core.Packed(entries)
        meta = (_core.ctypes.c_int * 4)()
        code = self._lib.blm_step_fill(self._h, packed.n, packed.slots, packed.counts, packed.tokens, packed.want_counts,
                                       packed.wants, pad_seqs, pad_tokens, width, out_ptr, capacity, meta, int(vocab))
        if code:
            _raise(code)
        return tuple(meta)

    def step_size(self, T: int, B: int, R: int, width: int) -> int:
        return int(self._lib.blm_step_size(len(self.groups), T, B, R, width))

    def pages_in_use(self) -> int:
        return sum(g.pool.n_pages - g.pool.n_free for g in self.groups)
