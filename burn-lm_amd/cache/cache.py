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
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import torch

from ..parts.base import KVNeed, StateNeed


class CacheError(RuntimeError):
    pass


class CacheFull(CacheError):
    """No slot or not enough pages are free; nothing was changed."""


class ContextOverflow(CacheError):
    """A sequence would grow past the longest context the cache was built for; nothing was changed."""

    def __init__(self, actual, maximum):
        super().__init__(f"context length exceeded: {actual} tokens, maximum {maximum}")
        self.actual, self.maximum = actual, maximum


class PagePool:
    """Free list of page numbers that knows which pages are out, so a page cannot be handed out
    twice or given back twice."""

    def __init__(self, n_pages: int):
        self.n_pages = n_pages
        self._free = list(range(n_pages - 1, -1, -1))
        self._out = set()

    @property
    def n_free(self):
        return len(self._free)

    def take(self, n: int) -> List[int]:
        if n > len(self._free):
            raise CacheFull(f"{n} pages wanted, {len(self._free)} free of {self.n_pages}")
        pages = [self._free.pop() for _ in range(n)]
        self._out.update(pages)
        return pages

    def give(self, pages: Sequence[int]) -> None:
        for p in pages:
            if p not in self._out:
                raise CacheError(f"page {p} given back but not handed out (freed twice?)")
        for p in pages:
            self._out.remove(p)
            self._free.append(p)


class KVGroup:
    def __init__(self, need: KVNeed, places: List[int], n_pages: int, page_size: int, dtype, device):
        self.need, self.places = need, places
        self.page_size = page_size
        self.pool = PagePool(n_pages)
        # [place in group, key|value, page, kv head, token in page * head_dim]; a key page is
        # [token][head_dim], a value page is stored transposed, [head_dim][token]
        self.storage = torch.empty(len(places), 2, n_pages, need.n_kv_heads, page_size * need.head_dim,
                                   dtype=dtype, device=device)
        self.tables: Dict[int, List[int]] = {}  # slot -> page of each page index (-1 once released)

    def pages_for(self, length: int) -> int:
        return (length + self.page_size - 1) // self.page_size

    def first_needed_page(self, length_after: int) -> int:
        """Pages wholly before the window of the *next* query are never read again."""
        if self.need.window <= 0:
            return 0
        first_key = max(0, length_after - self.need.window + 1)  # oldest key the next token may see
        return first_key // self.page_size


@dataclass
class _Seq:
    length: int = 0


class KVView:
    """What an attention-like mixer gets for its place in the order: the two storage planes, the
    page geometry, and (per step) the page table of the step's sequences."""

    def __init__(self, group: KVGroup, group_index: int, plane: int, store: bool):
        self.group_index, self.store = group_index, store
        n_pages, nkv, hd = group.storage.shape[2], group.need.n_kv_heads, group.need.head_dim
        self.k = group.storage[plane, 0].view(n_pages, nkv, group.page_size, hd)
        self.v = group.storage[plane, 1].view(n_pages, nkv, hd, group.page_size)
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
    """needs[i] is what place i of the layer order keeps (KVNeed, StateNeed or None);
    reads_from[i] is the earlier place whose keys and values place i reads instead of keeping
    its own (or None)."""

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
        self.views: List = [None] * len(needs)
        self.state_tensors: List[torch.Tensor] = []
        by_need: Dict[KVNeed, List[int]] = {}
        for i, need in enumerate(needs):
            if reads_from[i] is not None:
                continue
            if isinstance(need, KVNeed):
                by_need.setdefault(need, []).append(i)
        for need, places in by_need.items():
            g = KVGroup(need, places, self.n_pages, page_size, dtype, device)
            gi = len(self.groups)
            self.groups.append(g)
            for plane, i in enumerate(places):
                self.views[i] = KVView(g, gi, plane, store=True)
        for i, need in enumerate(needs):
            src = reads_from[i]
            if src is not None:
                if not (0 <= src < i) or reads_from[src] is not None or not isinstance(self.views[src], KVView):
                    raise CacheError(f"place {i} of the layer order reads the cache of place {src}, which must be "
                                     f"an earlier place that keeps keys and values of its own")
                sv = self.views[src]
                if isinstance(need, KVNeed) and (need.n_kv_heads, need.head_dim) != (sv.need.n_kv_heads, sv.need.head_dim):
                    raise CacheError(f"place {i} cannot read the cache of place {src}: head counts or sizes differ")
                g = self.groups[sv.group_index]
                self.views[i] = KVView(g, sv.group_index, g.places.index(src), store=False)
            elif isinstance(need, StateNeed):
                t = torch.zeros(max_seqs, *need.shape, dtype=need.dtype, device=device)
                self.state_tensors.append(t)
                self.views[i] = StateView(t)
        self._free_slots = list(range(max_seqs - 1, -1, -1))
        self._seqs: Dict[int, _Seq] = {}

    # ---- slots -----------------------------------------------------------------------------
    @property
    def free_slots(self):
        return len(self._free_slots)

    @property
    def live_slots(self):
        return sorted(self._seqs)

    def open(self) -> int:
        if not self._free_slots:
            raise CacheFull(f"all {self.max_seqs} sequence slots are in use")
        slot = self._free_slots.pop()
        self._seqs[slot] = _Seq()
        for g in self.groups:
            g.tables[slot] = []
        for t in self.state_tensors:
            t[slot].zero_()
        return slot

    def close(self, slot: int) -> None:
        if slot not in self._seqs:
            raise CacheError(f"slot {slot} is not open (closed twice?)")
        for g in self.groups:
            g.pool.give([p for p in g.tables.pop(slot) if p >= 0])
        del self._seqs[slot]
        self._free_slots.append(slot)

    def length(self, slot: int) -> int:
        try:
            return self._seqs[slot].length
        except KeyError:
            raise CacheError(f"slot {slot} is not open") from None

    def room(self, slot: int) -> int:
        return self.max_context - self.length(slot)

    # ---- growth ----------------------------------------------------------------------------
    def reserve(self, growth: Sequence) -> None:
        """growth: (slot, n_new) pairs of one step.  Hands out the pages all of them need, or
        raises before anything changed."""
        seen = set()
        wanted = [0] * len(self.groups)
        for slot, n in growth:
            if slot in seen:
                raise CacheError(f"slot {slot} appears twice in one step")
            seen.add(slot)
            length = self.length(slot)
            if n <= 0:
                raise CacheError(f"slot {slot}: a step must bring at least one token")
            if length + n > self.max_context:
                raise ContextOverflow(length + n, self.max_context)
            for gi, g in enumerate(self.groups):
                wanted[gi] += g.pages_for(length + n) - len(g.tables[slot])
        for gi, g in enumerate(self.groups):
            if wanted[gi] > g.pool.n_free:
                raise CacheFull(f"the step needs {wanted[gi]} more pages of {self.page_size} tokens, "
                                f"{g.pool.n_free} are free of {g.pool.n_pages}")
        for slot, n in growth:
            length = self._seqs[slot].length
            for g in self.groups:
                more = g.pages_for(length + n) - len(g.tables[slot])
                if more > 0:
                    g.tables[slot].extend(g.pool.take(more))

    def advance(self, slot: int, n: int) -> None:
        """The step that reserved n tokens for the slot has run: the sequence is n longer."""
        seq = self._seqs[slot]
        seq.length += n
        for g in self.groups:
            first = g.first_needed_page(seq.length)
            table = g.tables[slot]
            gone = [table[i] for i in range(min(first, len(table))) if table[i] >= 0]
            if gone:
                g.pool.give(gone)
                for i in range(min(first, len(table))):
                    table[i] = -1

    def page_table(self, group_index: int, slots: Sequence[int], width: int) -> List[List[int]]:
        g = self.groups[group_index]
        rows = []
        for s in slots:
            t = g.tables[s] if s >= 0 else []
            if len(t) > width:
                raise CacheError("page table wider than asked for")
            rows.append(t + [-1] * (width - len(t)))
        return rows

    def pages_in_use(self) -> int:
        return sum(g.pool.n_pages - g.pool.n_free for g in self.groups)
