"""The generation loop above the step function.

Requests (token-id prompts) are served in batches that start together: all prompts of a batch in
one step, then one token for each live sequence per step.  A sequence ends at a stop token, at
its ``sample_len``, or at the end of the context; it then leaves the batch and gives its slot
and pages back, while the others go on.  When a batch is done the next one starts, on the same
slots, until every request is served.

The reference's loop is ``Llama::generate`` (crates/burn-lm-llama/src/generation/generate.rs:
37-110): one request, ``reset()`` first, prompt step, then one token per step up to
``sample_len``, with the stop token found asynchronously by a decoder thread
(generation/context.rs:142-170) so that one more step may run.  Like the reference the stop token
is counted and returned but is not text.  Where the reference slides its window when the
context is full (nn/transformer.rs:156-163), a sequence here ends with the reason ``length``.

A batch's prompts run in one step while they are at most ``prompt_budget`` tokens together; a
larger batch is fed in several steps of that many tokens (the step function takes a prompt in
pieces; a sequence's last piece asks for its logits), so that the activations of a step stay
bounded whatever the requests bring.  A request that could not run even with the whole cache to
itself ends with ``finish_reason="error"`` and the others run, as a request whose prompt is longer
than the context does (crates/burn-lm-llama/src/nn/transformer.rs:148-154 and
server/llama3.rs:476-478 answer one request with an error and stay usable).

The loop needs of its engine only ``open / close / step / length / max_context / cache`` and of
its sampler only ``pick``, so its decisions are testable without a GPU.  With those alone the
stop is seen on the host in the same step and no extra step runs.  If the engine also has
``step_ahead`` and the sampler ``pick_device``, the loop keeps the GPU busy while the host reads
tokens: the tokens picked for a step stay on the GPU and feed the next step at once, and the
host looks at them one step late.  A sequence that met a stop token has then, as in the
reference, run one step too many, whose token is dropped; ends that are known beforehand
(``sample_len``, the end of the context) cost no extra step.  The tokens are the same either way.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, List, Optional, Sequence

from ..cache import core as _core
from .stats import Stats


class ContextLengthExceeded(ValueError):
    """Mirrors InferenceError::ContextLengthExceeded (crates/burn-lm-inference/src/errors.rs)."""

    def __init__(self, actual, maximum):
        super().__init__(f"Input sequence length ({actual} tokens) exceeds maximum context window ({maximum} "
                         f"tokens). Please shorten your input or increase the maximum context window.")
        self.actual, self.maximum = actual, maximum


@dataclass
class Generation:
    request: int
    prompt_len: int
    tokens: List[int] = field(default_factory=list)
    finish_reason: Optional[str] = None  # "stop" | "length" | "error"
    error: Optional[str] = None


# Most prompt tokens that one step runs; a batch whose prompts are more is fed in several steps.
PROMPT_BUDGET = 16384


def plan_batches(prompt_lens: Sequence[int], sample_len: int, batch_size: int, max_context: int,
                 page_size: int, n_pages: int, n_slots: int, unfit: Optional[List[int]] = None) -> List[List[int]]:
    """Cuts the requests, in order, into batches that fit: at most batch_size sequences and slots,
    and pages enough for every sequence of the batch to reach its longest possible length (decided
    by the native core, blm_plan_batches).  A request that needs more pages than the cache has is in
    no batch; its index is appended to ``unfit`` if that list is given."""
    n = len(prompt_lens)
    if n == 0:
        return []
    batch_of = (_core.ctypes.c_int * n)()
    n_batches = _core.library().blm_plan_batches(n, _core.ints(list(prompt_lens)), int(sample_len), int(batch_size),
                                                 int(max_context), int(page_size), int(n_pages), int(n_slots), batch_of)
    batches = [[] for _ in range(n_batches)]
    for i in range(n):
        if batch_of[i] >= 0:
            batches[batch_of[i]].append(i)
        elif unfit is not None:
            unfit.append(i)
    return batches


def plan_prompt_steps(prompt_lens: Sequence[int], budget: int) -> List[List[tuple]]:
    """The prompts of one batch as steps of at most `budget` tokens: per step a list of (sequence,
    first token, number of tokens), sequences in order, a prompt cut wherever a step is full (decided
    by the native core, blm_plan_prompt_steps)."""
    n = len(prompt_lens)
    if budget <= 0:
        raise ValueError("the prompt budget must be positive")
    most = n + sum(prompt_lens) // budget + 1
    arrays = [(_core.ctypes.c_int * most)() for _ in range(4)]
    pieces = _core.library().blm_plan_prompt_steps(n, _core.ints(list(prompt_lens)), int(budget), most, *arrays)
    if pieces < 0:
        raise ValueError("prompts must hold at least one token each")
    steps: List[List[tuple]] = []
    for p in range(pieces):
        if arrays[0][p] == len(steps):
            steps.append([])
        steps[-1].append((arrays[1][p], arrays[2][p], arrays[3][p]))
    return steps


def _cache_refusals():
    from ..cache.cache import CacheFull, ContextOverflow
    return (CacheFull, ContextOverflow)


class _Book:
    """The generation's bookkeeping in the native core (csrc/host/generation.h): how many tokens each
    request has, how long its sequence is, what a token means for it, who may run ahead."""
    GOES_ON, STOP, LENGTH, DROPPED = 0, 1, 2, -1

    def __init__(self, prompt_lens, sample_len, max_context, stop_ids):
        self._lib = _core.library()
        stops = sorted(stop_ids)
        self._h = self._lib.blm_gen_new(len(prompt_lens), _core.ints(list(prompt_lens)), int(sample_len), int(max_context),
                                        len(stops), _core.ints(stops))
        if not self._h:
            raise ValueError("bad sizes for a generation")
        self._buf = (_core.ctypes.c_int * max(1, len(prompt_lens)))()
        self._buf2 = (_core.ctypes.c_int * max(1, len(prompt_lens)))()

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.blm_gen_free(self._h)
            self._h = None

    def start(self, requests):
        if self._lib.blm_gen_start(self._h, len(requests), _core.ints(list(requests))):
            raise ValueError("a batch names a request that does not exist")

    def ahead_rows(self):
        n = self._lib.blm_gen_ahead_rows(self._h, self._buf)
        return self._buf[:n]

    def launched(self, rows):
        if self._lib.blm_gen_launched(self._h, len(rows), _core.ints(list(rows))):
            raise ValueError("a launched row is not a live entry")

    def take(self, tokens):
        """-> (entries that go on, what each entry's token means)"""
        n = len(tokens)
        going = self._lib.blm_gen_take(self._h, _core.ints(list(tokens)), self._buf)
        return going, self._buf[:n]

    def live(self):
        n = self._lib.blm_gen_live(self._h, self._buf, self._buf2)
        return self._buf[:n], self._buf2[:n]


def run_prompts(engine, slots: Sequence[int], prompts: Sequence[Sequence[int]], budget: int):
    """Feeds the prompts of a batch, in steps of at most `budget` tokens.  -> (the logits after every
    prompt's last token, in the order of the prompts; the number of steps it took)."""
    if sum(len(p) for p in prompts) <= budget:
        return engine.step([(s, list(p), [len(p) - 1]) for s, p in zip(slots, prompts)]), 1
    steps = plan_prompt_steps([len(p) for p in prompts], budget)
    rows = [None] * len(prompts)
    for pieces in steps:
        ends = [k for k, first, count in pieces if first + count == len(prompts[k])]
        logits = engine.step([(slots[k], list(prompts[k][first:first + count]),
                               [count - 1] if first + count == len(prompts[k]) else []) for k, first, count in pieces])
        for r, k in enumerate(ends):
            rows[k] = logits[r].clone()     # a later step may write into the buffer these logits live in
    return _stack(rows), len(steps)


def _stack(rows):
    import torch
    return torch.stack(rows)


def generate(engine, prompts: Sequence[Sequence[int]], sampler, sample_len: int, stop_ids: Sequence[int] = (),
             batch_size: int = 8, on_token: Optional[Callable[[int, int], None]] = None,
             clock: Callable[[], float] = time.perf_counter, prompt_budget: int = PROMPT_BUDGET):
    """-> (list of Generation in request order, Stats).  ``on_token(request, token)`` is called
    for every generated token as soon as it is known (stop tokens included).  ``prompt_budget``: the
    most prompt tokens one step runs."""
    if sample_len < 0:
        raise ValueError("sample_len must be >= 0")
    if prompt_budget <= 0:
        raise ValueError("prompt_budget must be positive")
    stop = set(int(s) for s in stop_ids)
    results = [Generation(i, len(p)) for i, p in enumerate(prompts)]
    stats = Stats()
    t_start = clock()
    runnable = []
    for i, p in enumerate(prompts):
        if len(p) == 0:
            results[i].finish_reason, results[i].error = "error", "empty prompt"
        elif len(p) > engine.max_context:
            e = ContextLengthExceeded(len(p), engine.max_context)
            results[i].finish_reason, results[i].error = "error", str(e)
        elif sample_len == 0:
            results[i].finish_reason = "length"
        else:
            runnable.append(i)
    cache = engine.cache
    unfit: List[int] = []
    batches = plan_batches([len(prompts[i]) for i in runnable], sample_len, batch_size, engine.max_context,
                           cache.page_size, cache.n_pages, cache.max_seqs, unfit)
    for j in unfit:
        i = runnable[j]
        reach = min(len(prompts[i]) + sample_len, engine.max_context)
        results[i].finish_reason = "error"
        results[i].error = (f"the request may grow to {reach} tokens, which takes {-(-reach // cache.page_size)} pages of the "
                            f"cache; it has {cache.n_pages}")
    ahead = hasattr(engine, "step_ahead") and hasattr(sampler, "pick_device")
    book = _Book([len(p) for p in prompts], sample_len, engine.max_context, stop)
    reason_names = {_Book.STOP: "stop", _Book.LENGTH: "length"}
    queue = [[runnable[j] for j in batch] for batch in batches]
    while queue:
        ids = queue.pop(0)
        slot_of, open_slots = {}, set()

        def close(slot):
            open_slots.discard(slot)
            engine.close(slot)

        try:
            for i in ids:       # inside the try: a slot that cannot be had must not strand the ones already opened
                slot = engine.open()
                open_slots.add(slot)
                slot_of[i] = slot
            t0 = clock()
            try:
                logits, n_steps = run_prompts(engine, [slot_of[i] for i in ids], [prompts[i] for i in ids], prompt_budget)
            except _cache_refusals() as e:
                # The cache could not take the prompts after all (the planner counts the pages of one group of
                # layers; a cache may have several).  Nothing of the refused step has changed anything: the slots
                # go back, a batch of several is tried one request at a time, a single request ends with the error.
                for slot in list(open_slots):
                    close(slot)
                if len(ids) > 1:
                    queue[0:0] = [[i] for i in ids]
                else:
                    results[ids[0]].finish_reason, results[ids[0]].error = "error", str(e)
                continue
            picked = sampler.pick(logits, ids, [0] * len(ids))
            stats.prompt_tokens += sum(len(prompts[i]) for i in ids)
            stats.prompt_seconds += clock() - t0
            stats.steps += n_steps
            t0 = clock()
            from_prompt = True
            book.start(ids)
            live = list(ids)        # requests whose token is pending, in the order of the pending tokens
            while True:
                # the step after the one whose tokens are still on their way, for every sequence that
                # cannot end at that token for a reason known beforehand
                launched = None
                if ahead and hasattr(picked, "tokens"):
                    rows = book.ahead_rows()
                    if rows:
                        logits = engine.step_ahead([slot_of[live[k]] for k in rows], rows, picked)
                        if logits is not None:
                            book.launched(rows)
                            nxt = [live[k] for k in rows]
                            launched = sampler.pick_device(logits, nxt, [len(results[i].tokens) + 1 for i in nxt])
                            stats.steps += 1
                tokens = picked.tokens() if hasattr(picked, "tokens") else picked
                going, reasons = book.take(tokens)
                for i, tok, why in zip(live, tokens, reasons):
                    if why == _Book.DROPPED:    # it had ended before the step in flight: this token is ignored
                        continue
                    r = results[i]
                    r.tokens.append(tok)
                    stats.generated_tokens += 1
                    if not from_prompt:
                        stats.decode_tokens += 1
                    if on_token is not None:
                        on_token(i, tok)
                    if why != _Book.GOES_ON:
                        r.finish_reason = reason_names[why]
                        close(slot_of[i])
                from_prompt = False
                live, _ = book.live()
                if launched is not None:
                    picked = launched
                    if going == 0:
                        break
                    continue
                if not live:
                    break
                logits = engine.step([(slot_of[i], [results[i].tokens[-1]], [0]) for i in live])
                indices = [len(results[i].tokens) for i in live]
                picked = sampler.pick_device(logits, live, indices) if ahead else sampler.pick(logits, live, indices)
                stats.steps += 1
            stats.decode_seconds += clock() - t0
        except BaseException:
            for slot in list(open_slots):
                try:
                    engine.close(slot)
                except Exception:
                    pass
            raise
    stats.inference_seconds = clock() - t_start
    return results, stats
