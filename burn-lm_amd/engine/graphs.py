"""Steps replayed as HIP graphs.

A step is some hundred kernels; launched one by one from Python they cost more time than they run
as long as the step is small: every decode step, and prompts up to a few thousand tokens.  For
every shape of such a step (sequences rounded up to a bucket, tokens rounded up to a bucket,
page-table width rounded up to a bucket) the step is run once eagerly, then captured, and from then
on replayed: the host only refreshes one int32 buffer (tokens, positions, page tables) and
launches the graph.  Two kinds of step are recorded: decode steps (one token per sequence, its
logits wanted) and prompt steps (any number of tokens per sequence, the last one's logits wanted).

A shape is recorded the second time it is met (a shape met once is not worth a graph), right after
it has run once more eagerly *at the bucket's own size* (all padding), so that every kernel and
library handle the recording needs exists beforehand.  At most ``MAX_GRAPHS`` shapes are kept; the
one replayed longest ago makes room for a new one (a recorded shape holds its index and logits
buffers and its share of the graphs' memory pool).

Places of the bucket that nothing fills are padding: padding tokens belong to no sequence (index
-1), so they write no cache; padding sequences bring no token; their rows are dropped.  The kernels
compute every row on its own, so padding changes no result.  Only models whose parts all declare
``graph_safe`` are replayed this way, and no memset node is recorded (buffers are cleared, where
needed, by kernels).
"""
from __future__ import annotations

import ctypes
import gc
import weakref
from typing import Dict, Tuple

import torch

from ..cache import core as _core
from .batch import Step

BATCH_BUCKETS = (1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128)
MAX_GRAPHS = 48         # recorded shapes kept at a time
RECORD_AT_SIGHT = 2     # a shape is recorded when it is met for this many-th time


def batch_bucket(n: int):
    for b in BATCH_BUCKETS:
        if n <= b:
            return b
    return None


# prompt steps: total tokens of the step, and at most this many sequences (a step's attention
# launches blocks for bucket sequences x bucket tokens; beyond these sizes the launches are no
# longer what a step's time goes to).  No bucket of 192: the library's products are slower at 192
# rows than at 256 (a 160-token prompt at the Llama-3.2-3B shape: 4.9 ms padded to 192, 4.3 to 256).
TOKEN_BUCKETS = (64, 128, 256, 384, 512, 768, 1024, 1536, 2048)
PROMPT_MAX_SEQS = 16


def token_bucket(n: int):
    for b in TOKEN_BUCKETS:
        if n <= b:
            return b
    return None


_BATCH_BUCKETS = _core.ints(BATCH_BUCKETS)
_TOKEN_BUCKETS = _core.ints(TOKEN_BUCKETS)


def width_bucket(pages: int, max_width: int) -> int:
    w = 8
    while w < pages:
        w *= 2
    return min(w, max(max_width, 1))


_LIB = _core.library


class _Captured:
    """One recorded shape: B sequences, T tokens (T = 0: a decode step, one token per sequence),
    page tables W wide."""

    def __init__(self, engine, B: int, T: int, W: int, pool):
        cache, dev = engine.cache, engine.rt.device
        G = len(cache.groups)
        self.B, self.T, self.W = B, T, W
        self.decode = T == 0
        NT = B if self.decode else T           # tokens of the recorded step
        self.copied = None
        n = 3 * NT + 4 * B + 1 + G * B * W     # the step's index arrays ...
        self.src_at = n                        # ... and behind them, for run_ahead, where each row's token comes from
        self.cell_at = (n + B + 1) // 2 * 2    # ... and the address of the array they come from (8 bytes, aligned)
        self.host = torch.zeros(self.cell_at + 2, dtype=torch.int32).pin_memory()
        self.host_np = self.host.numpy()
        self.host_np[n: n + B] = -1            # no row's token comes from the device
        self.host_cell = self.host_np[self.cell_at: self.cell_at + 2].view("int64")
        self.dev = torch.zeros(self.cell_at + 2, dtype=torch.int32, device=dev)
        self.ahead_rows = 0                    # rows of the host image that the last run_ahead pointed at the device
        # an embedding that can take tokens from the device does so inside the recorded step; for
        # another one they are gathered into token_ids by a launch before the replay
        self.folded = self.decode and hasattr(engine.model.embedding, "forward_from")
        o = 0

        def take(k):
            nonlocal o
            v = self.dev[o:o + k]
            o += k
            return v

        token_ids, positions, token_seq, seq_slots = take(NT), take(NT), take(NT), take(B)
        cu, after, rows = take(B + 1), take(B), take(B)
        tables = {gi: take(B * W).view(B, W) for gi in range(G)}
        self.src_rows = take(B)
        span = min(W * cache.page_size, cache.max_context)
        self.step = Step(n_tokens=NT, n_seqs=B, n_wanted=B, token_ids=token_ids, positions=positions,
                         token_seq=token_seq, seq_slots=seq_slots, cu_seqlens=cu, lens_after=after, want_rows=rows,
                         block_tables=tables, max_new=1 if self.decode else T, max_position=span - 1,
                         max_len_after=span, is_decode=self.decode, host_slots=[], host_new=[])
        if self.folded:
            self.step.token_source = (self.src_rows, self.dev[self.cell_at: self.cell_at + 2].view(torch.int64))
        self.fill(None, cache)     # all padding: valid contents while capturing
        self.dev.copy_(self.host)
        engine.model.forward(self.step, cache)      # once eagerly at the bucket's size: what the recording meets exists
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

    def fill(self, entries, cache):
        """Host image of the index buffer for these packed (slot, tokens, [last]) entries, the rest padding
        (None: all padding);
        written by the native core straight into the pinned buffer."""
        B, W = self.B, self.W
        NT = B if self.decode else self.T
        if entries is not None:
            cache.fill_step(entries, B, NT, W, self.host.data_ptr(), self.src_at)
            return
        # all padding (used while recording): token 0, position 0, no sequence, no slot, no pages
        flat = [0] * NT + [0] * NT + [-1] * NT + [-1] * B + [0] * (B + 1) + [0] * B + [0] * B
        flat += [-1] * (len(cache.groups) * B * W)
        self.host[: self.src_at].copy_(torch.tensor(flat, dtype=torch.int32))

    def run(self, entries, cache):
        if self.copied is not None:
            self.copied.synchronize()      # the last copy out of the host image must be over before it changes
        self.fill(entries, cache)
        if self.ahead_rows:
            self.host_np[self.src_at: self.src_at + self.ahead_rows] = -1
            self.ahead_rows = 0
        self.dev.copy_(self.host, non_blocking=True)
        self.copied = torch.cuda.Event()
        self.copied.record()
        self.graph.replay()
        return self.logits[: entries.n].clone()   # the graph's own output buffer is overwritten by the next replay

    def run_ahead(self, packed, rows, tokens_dev, cache):
        """Like run() for a decode step, but row i's token is tokens_dev[rows[i]], taken on the device:
        the host need not have seen the tokens of the step before.  The logits come back without a copy."""
        if self.copied is not None:
            self.copied.synchronize()
        n = packed.n
        self.fill(packed, cache)
        self.host_np[self.src_at: self.src_at + n] = rows
        if self.ahead_rows > n:
            self.host_np[self.src_at + n: self.src_at + self.ahead_rows] = -1
        self.ahead_rows = n
        self.host_cell[0] = tokens_dev.data_ptr()
        self.dev.copy_(self.host, non_blocking=True)
        self.copied = torch.cuda.Event()
        self.copied.record()
        if not self.folded:
            torch.index_select(tokens_dev, 0, self.src_rows[:n], out=self.step.token_ids[:n])
        self.graph.replay()
        return self.logits[:n]      # the graph's own buffer: good until the next replay of this shape


class StepGraphs:
    def __init__(self, engine):
        # a weak reference: the engine owns this object, and a cycle would leave the graphs to the
        # cyclic collector, which may run at any time (see the note on capture above)
        self._engine = weakref.ref(engine)
        self.captured: Dict[Tuple[int, int, int], _Captured] = {}     # in order of last use, oldest first
        self.sightings: Dict[Tuple[int, int, int], int] = {}
        self.pool = None
        self.enabled = all(p.graph_safe for p in engine.model.all_parts())
        self.replays = 0
        self.evicted = 0

    def key_for(self, packed):
        """Bucket key (sequences, tokens or 0 for a decode step, table width) of a step (its packed
        entries), or None if the step cannot be replayed from a graph; decided by the native core."""
        if not self.enabled:
            return None
        cache = self._engine().cache
        lengths = cache.lengths_of(packed)
        key = (ctypes.c_int * 3)()
        _LIB().blm_step_key(packed.n, packed.counts, lengths, packed.want_counts, packed.wants, len(BATCH_BUCKETS),
                            _BATCH_BUCKETS, len(TOKEN_BUCKETS), _TOKEN_BUCKETS, PROMPT_MAX_SEQS, cache.page_size,
                            cache.table_width, key)
        return None if key[0] < 0 else (key[0], key[1], key[2])

    def run(self, key, entries):
        """Replays the step if its shape has been captured; returns None if it must run eagerly
        (the first time a shape is met; it is captured right after that run)."""
        c = self._use(key)
        if c is None:
            return None
        self.replays += 1
        return c.run(entries, self._engine().cache)

    def _use(self, key):
        """The recorded shape, moved to the young end of the order of use; None if it is not recorded."""
        c = self.captured.pop(key, None)
        if c is not None:
            self.captured[key] = c
        return c

    def run_ahead(self, key, packed, rows, tokens_dev):
        """Replays a recorded decode shape with the tokens taken on the device; None if it is not recorded."""
        c = self._use(key)
        if c is None:
            return None
        self.replays += 1
        return c.run_ahead(packed, rows, tokens_dev, self._engine().cache)

    def after_eager(self, key):
        """The shape has just run eagerly.  Met for the second time it is recorded for the times to
        come; the shape used longest ago goes if the table is full."""
        if key in self.captured:
            return
        self.sightings[key] = self.sightings.get(key, 0) + 1
        if self.sightings[key] < RECORD_AT_SIGHT:
            return
        if self.pool is None:
            self.pool = torch.cuda.graph_pool_handle()
        while len(self.captured) >= MAX_GRAPHS:
            oldest = next(iter(self.captured))
            torch.cuda.synchronize()        # nothing of the old shape is still running when its buffers go
            del self.captured[oldest]
            self.sightings.pop(oldest, None)
            self.evicted += 1
        self.captured[key] = _Captured(self._engine(), key[0], key[1], key[2], self.pool)
