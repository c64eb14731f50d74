"""The step function: a model, its cache, and one call that runs exactly the tokens it is given.

``step(entries)`` takes, per sequence, its slot, its next tokens and the places among them whose
logits are wanted.  The sequences of a call may have different lengths and different pasts; the
tokens run as one packed batch, each attending to its own sequence's cache, and the logits of
the wanted rows come back as float32 ``[wanted, vocab]`` in the order of the entries and of
their ``want`` lists.  Position of the t-th new token of a sequence = tokens it already holds + t
(crates/burn-lm-llama/src/nn/pos_encoding.rs:66-79).  Everything is checked before anything
changes: a refused step leaves cache and sequences as they were.  One iteration body of the
reference's loop (crates/burn-lm-llama/src/generation/generate.rs:66-85) is one such step.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch

from ..cache.cache import Cache, CacheError
from ..cache.core import Packed


class StepError(ValueError):
    pass


class Engine:
    def __init__(self, model, rt, max_tokens: int, max_seqs: Optional[int] = None,
                 max_context: Optional[int] = None, page_size: int = 64, graphs: bool = True):
        self.model, self.rt = model, rt
        plan_max = model.plan.max_positions
        n_pages = (max_tokens + page_size - 1) // page_size
        max_context = min(max_context or plan_max, plan_max, n_pages * page_size)
        max_seqs = max_seqs or min(n_pages, 4096)
        self.cache = Cache(model.cache_needs(), model.reads_from(), max_tokens=n_pages * page_size,
                           max_seqs=max_seqs, max_context=max_context, page_size=page_size,
                           dtype=rt.dtype, device=rt.device)
        model.prepare_positions(max_context)
        self.max_context = max_context
        self.vocab_size = model.vocab_size
        from .graphs import StepGraphs
        self.graphs = StepGraphs(self) if graphs else None

    # ---- sequences ---------------------------------------------------------------------------
    def open(self) -> int:
        return self.cache.open()

    def close(self, slot: int) -> None:
        self.cache.close(slot)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    def clear(self) -> None:
        """Close every live sequence."""
        for s in self.cache.live_slots:
            self.cache.close(s)

    # ---- the step ----------------------------------------------------------------------------
    def _pack(self, entries):
        """The step's entries as flat arrays for the native core, everything about them checked there:
        slots open, at least one token per sequence, tokens inside the vocabulary, wanted places inside
        each sequence's tokens.  StepError before anything changes."""
        try:
            packed = Packed(entries)
        except (TypeError, OverflowError, ValueError) as e:
            raise StepError(f"a step's slots, tokens and wanted places must be integers that fit 32 bits: {e}") from None
        if packed.n == 0:
            raise StepError("a step needs at least one sequence")
        try:
            self.cache.check_step(packed, self.vocab_size)
        except CacheError as e:
            raise StepError(str(e)) from None
        return packed

    def step(self, entries: Sequence[Tuple[int, Sequence[int], Sequence[int]]]) -> Optional[torch.Tensor]:
        packed = self._pack(entries)
        self.cache.reserve_step(packed)  # raises before any change
        key = self.graphs.key_for(packed) if self.graphs is not None else None
        logits = self.graphs.run(key, packed) if key is not None else None
        if logits is None:
            logits = self.model.forward(self.build_step(packed), self.cache)
            if key is not None:
                self.graphs.after_eager(key)
        self.cache.advance_step(packed)
        return logits

    def step_ahead(self, slots: Sequence[int], rows: Sequence[int], picked) -> Optional[torch.Tensor]:
        """One more token for each of the sequences in slots, without the host knowing the tokens
        yet: sequence i's token is ``picked.device[rows[i]]`` (what a sampler left on the GPU for
        the step before).  Returns the logits of these tokens, or None, with nothing changed, if
        the step's shape has no recorded graph (the caller then reads the tokens and uses step()).
        The logits are the recorded graph's own buffer: work queued on the stream before the next
        step (a sampler's pick) reads them safely, a caller that keeps them longer must copy them."""
        if self.graphs is None:
            return None
        if picked.device.dtype != torch.int32 or not picked.device.is_contiguous() or picked.device.dim() != 1:
            raise StepError("step_ahead takes the picked tokens as a contiguous int32 vector on the device")
        n_picked = picked.device.shape[0]
        if not slots or len(rows) != len(slots) or min(rows) < 0 or max(rows) >= n_picked:
            raise StepError("step_ahead needs one row of the picked tokens for every sequence")
        packed = Packed.one_token_each(slots)
        key = self.graphs.key_for(packed)
        if key is None or key not in self.graphs.captured:
            return None
        self.cache.reserve_step(packed)  # raises before any change
        logits = self.graphs.run_ahead(key, packed, rows, picked.device)
        self.cache.advance_step(packed)
        return logits

    def build_step(self, entries):
        """The eager step's index arrays on the device; entries: (slot, tokens, want) tuples or a Packed."""
        from .batch import build_step
        return build_step(entries, self.cache, self.rt.device)
