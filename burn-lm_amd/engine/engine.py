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

import operator
from typing import Optional, Sequence, Tuple

import torch

from ..cache.cache import Cache


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
    @staticmethod
    def _integers(slot, what, values):
        """values as Python integers; anything that is no integer (a float, a string, a bool) is refused
        as such, numpy's and torch's integer scalars are taken."""
        out = []
        for v in values:
            if isinstance(v, bool):
                raise StepError(f"slot {slot}: {what} {v!r} is a {type(v).__name__}, not an integer")
            try:
                out.append(operator.index(v))
            except TypeError:
                raise StepError(f"slot {slot}: {what} {v!r} is a {type(v).__name__}, not an integer") from None
        return out

    def _check(self, entries):
        if not entries:
            raise StepError("a step needs at least one sequence")
        V = self.vocab_size
        for slot, tokens, want in entries:
            n = len(tokens)
            if n == 0:
                raise StepError(f"slot {slot}: a step must bring at least one token per sequence")
            for t in tokens:
                if not 0 <= t < V:
                    raise StepError(f"slot {slot}: token {t!r} is outside the vocabulary of {V}")
            for w in want:
                if not 0 <= w < n:
                    raise StepError(f"slot {slot}: wanted place {w!r} is outside this step's {n} tokens")

    def step(self, entries: Sequence[Tuple[int, Sequence[int], Sequence[int]]]) -> Optional[torch.Tensor]:
        self.rt.check_fault()
        entries = [(int(s), self._integers(s, "token", t), self._integers(s, "wanted place", w)) for s, t, w in entries]
        self._check(entries)
        lengths = [self.cache.length(s) for s, _, _ in entries]
        self.cache.reserve([(s, len(t)) for s, t, _ in entries])  # raises before any change
        key = self.graphs.key_for(entries, lengths) if self.graphs is not None else None
        logits = self.graphs.run(key, entries) if key is not None else None
        if logits is None:
            step = self.build_step(entries, lengths)
            logits = self.model.forward(step, self.cache)
            if key is not None:
                self.graphs.after_eager(key)
        for s, t, _ in entries:
            self.cache.advance(s, len(t))
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
        slots = [int(s) for s in slots]
        rows = [int(r) for r in rows]
        if not slots or len(rows) != len(slots) or any(not 0 <= r < picked.device.shape[0] for r in rows):
            raise StepError("step_ahead needs one row of the picked tokens for every sequence")
        lengths = [self.cache.length(s) for s in slots]
        key = self.graphs.key_for([(s, [0], [0]) for s in slots], lengths)
        if key is None or key not in self.graphs.captured:
            return None
        self.cache.reserve([(s, 1) for s in slots])  # raises before any change
        logits = self.graphs.run_ahead(key, slots, rows, picked.device)
        for s in slots:
            self.cache.advance(s, 1)
        return logits

    def build_step(self, entries, lengths):
        from .batch import build_step
        return build_step(entries, lengths, self.cache, self.rt.device)
