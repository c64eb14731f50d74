"""Decode steps replayed as HIP graphs.

A decode step is some hundred small kernels; launched one by one from Python they cost more time
than they run.  For every shape of decode step (sequences rounded up to a bucket, page-table width
rounded up to a bucket) the step is run once eagerly, then captured, and from then on replayed: the
host only refreshes one int32 buffer (tokens, positions, page tables) and launches the graph.

Places of the bucket that no sequence fills are padding: their sequence index is -1, so they write
no cache and their rows are dropped; the kernels compute every row on its own, so padding changes
no result.  Only models whose parts all declare ``graph_safe`` are replayed this way, and no memset
node is recorded (buffers are cleared, where needed, by kernels).
"""
from __future__ import annotations

import gc
import weakref
from typing import Dict, Tuple

import torch

from .batch import Step

BATCH_BUCKETS = (1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128)


def batch_bucket(n: int):
    for b in BATCH_BUCKETS:
        if n <= b:
            return b
    return None


def width_bucket(pages: int, max_width: int) -> int:
    w = 8
    while w < pages:
        w *= 2
    return min(w, max(max_width, 1))


class _Captured:
    def __init__(self, engine, B: int, W: int, pool):
        cache, dev = engine.cache, engine.rt.device
        G = len(cache.groups)
        self.B, self.W = B, W
        self.copied = None
        n = 7 * B + 1 + G * B * W          # the step's index arrays ...
        self.src_at = n                    # ... and behind them, for run_ahead, where each row's token comes from
        self.host = torch.zeros(n + B, dtype=torch.int32).pin_memory()
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(n + B, dtype=torch.int32, device=dev)
        o = 0

        def take(k):
            nonlocal o
            v = self.dev[o:o + k]
            o += k
            return v

        token_ids, positions, token_seq, seq_slots = take(B), take(B), take(B), take(B)
        cu, after, rows = take(B + 1), take(B), take(B)
        tables = {gi: take(B * W).view(B, W) for gi in range(G)}
        self.src_rows = take(B)
        span = min(W * cache.page_size, cache.max_context)
        self.step = Step(n_tokens=B, n_seqs=B, n_wanted=B, token_ids=token_ids, positions=positions,
                         token_seq=token_seq, seq_slots=seq_slots, cu_seqlens=cu, lens_after=after, want_rows=rows,
                         block_tables=tables, max_new=1, max_position=span - 1, max_len_after=span, is_decode=True,
                         host_slots=[], host_new=[])
        self.fill([], [], cache)       # all padding: valid contents while capturing
        self.dev.copy_(self.host)
        self.graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()
        # No garbage collection while the capture is open: a collected object that owns GPU memory or
        # another graph would free it in the middle of the capture, which HIP answers with an abort.
        was_enabled = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(self.graph, pool=pool):
                self.logits = engine.model.forward(self.step, cache)
        finally:
            if was_enabled:
                gc.enable()
        torch.cuda.synchronize()

    def fill(self, entries, lengths, cache):
        """Host image of the index buffer for these (slot, [token], [0]) entries, the rest padding;
        written by the native core straight into the pinned buffer."""
        B, W = self.B, self.W
        if entries:
            cache.fill_step(entries, B, W, self.host.data_ptr(), self.src_at)
            return
        # all padding (used while recording): token 0, position 0, no sequence, no slot, no pages
        flat = [0] * B + [0] * B + [-1] * B + [-1] * B + list(range(B + 1)) + [0] * B + list(range(B))
        flat += [-1] * (len(cache.groups) * B * W)
        self.host[: self.src_at].copy_(torch.tensor(flat, dtype=torch.int32))

    def run(self, entries, lengths, cache):
        if self.copied is not None:
            self.copied.synchronize()      # the last copy out of the host image must be over before it changes
        self.fill(entries, lengths, cache)
        self.dev.copy_(self.host, non_blocking=True)
        self.copied = torch.cuda.Event()
        self.copied.record()
        self.graph.replay()
        return self.logits[: len(entries)].clone()   # the graph's own output buffer is overwritten by the next replay

    def run_ahead(self, slots, rows, tokens_dev, cache):
        """Like run(), but row i's token is tokens_dev[rows[i]], taken on the device: the host
        need not have seen the tokens of the step before.  The logits come back without a copy."""
        if self.copied is not None:
            self.copied.synchronize()
        n = len(slots)
        self.fill([(s, [0], [0]) for s in slots], None, cache)
        self.host_np[self.src_at: self.src_at + n] = rows
        self.dev.copy_(self.host, non_blocking=True)
        self.copied = torch.cuda.Event()
        self.copied.record()
        torch.index_select(tokens_dev, 0, self.src_rows[:n], out=self.step.token_ids[:n])
        self.graph.replay()
        return self.logits[:n]      # the graph's own buffer: good until the next replay of this shape


class DecodeGraphs:
    def __init__(self, engine):
        # a weak reference: the engine owns this object, and a cycle would leave the graphs to the
        # cyclic collector, which may run at any time (see the note on capture above)
        self._engine = weakref.ref(engine)
        self.captured: Dict[Tuple[int, int], _Captured] = {}
        self.seen = set()
        self.pool = None
        self.enabled = all(p.graph_safe for p in engine.model.all_parts())
        self.replays = 0

    def key_for(self, entries, lengths):
        """Bucket key of a decode step, or None if the step cannot be replayed from a graph."""
        if not self.enabled or any(len(t) != 1 or w != [0] for _, t, w in entries):
            return None
        B = batch_bucket(len(entries))
        if B is None:
            return None
        cache = self._engine().cache
        pages = (max(lengths) + 1 + cache.page_size - 1) // cache.page_size
        return B, width_bucket(pages, cache.table_width)

    def run(self, key, entries, lengths):
        """Replays the step if its shape has been captured; returns None if it must run eagerly
        (the first time a shape is met; it is captured right after that run)."""
        c = self.captured.get(key)
        if c is None:
            return None
        self.replays += 1
        return c.run(entries, lengths, self._engine().cache)

    def run_ahead(self, key, slots, rows, tokens_dev):
        """Replays a recorded shape with the tokens taken on the device; None if it is not recorded."""
        c = self.captured.get(key)
        if c is None:
            return None
        self.replays += 1
        return c.run_ahead(slots, rows, tokens_dev, self._engine().cache)

    def after_eager(self, key):
        """The shape has just run eagerly (so every kernel and library handle it needs exists):
        capture it for the next time."""
        if key in self.captured:
            return
        if self.pool is None:
            self.pool = torch.cuda.graph_pool_handle()
        self.captured[key] = _Captured(self._engine(), key[0], key[1], self.pool)
