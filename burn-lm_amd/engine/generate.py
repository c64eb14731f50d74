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


def _pages(n_tokens, page):
    return (n_tokens + page - 1) // page


def plan_batches(prompt_lens: Sequence[int], sample_len: int, batch_size: int, max_context: int,
                 page_size: int, n_pages: int, n_slots: int) -> List[List[int]]:
    """Cuts the requests, in order, into batches that fit: at most batch_size sequences and slots,
    and pages enough for every sequence of the batch to reach its longest possible length."""
    batches, cur, used = [], [], 0
    for i, n in enumerate(prompt_lens):
        need = _pages(min(n + sample_len, max_context), page_size)
        if cur and (len(cur) >= min(batch_size, n_slots) or used + need > n_pages):
            batches.append(cur)
            cur, used = [], 0
        cur.append(i)
        used += need
    if cur:
        batches.append(cur)
    return batches


def generate(engine, prompts: Sequence[Sequence[int]], sampler, sample_len: int, stop_ids: Sequence[int] = (),
             batch_size: int = 8, on_token: Optional[Callable[[int, int], None]] = None,
             clock: Callable[[], float] = time.perf_counter):
    """-> (list of Generation in request order, Stats).  ``on_token(request, token)`` is called
    for every generated token as soon as it is known (stop tokens included)."""
    if sample_len < 0:
        raise ValueError("sample_len must be >= 0")
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
    batches = plan_batches([len(prompts[i]) for i in runnable], sample_len, batch_size, engine.max_context,
                           cache.page_size, cache.n_pages, cache.max_seqs)
    ahead = hasattr(engine, "step_ahead") and hasattr(sampler, "pick_device")
    for batch in batches:
        ids = [runnable[j] for j in batch]
        live, open_slots = [], set()

        def close(slot):
            open_slots.discard(slot)
            engine.close(slot)

        try:
            for i in ids:       # inside the try: a slot that cannot be had must not strand the ones already opened
                slot = engine.open()
                open_slots.add(slot)
                live.append((i, slot))
            t0 = clock()
            logits = engine.step([(slot, list(prompts[i]), [len(prompts[i]) - 1]) for i, slot in live])
            picked = sampler.pick(logits, [i for i, _ in live], [0] * len(live))
            stats.prompt_tokens += sum(len(prompts[i]) for i, _ in live)
            stats.prompt_seconds += clock() - t0
            stats.steps += 1
            t0 = clock()
            from_prompt = True
            dropped = set()     # requests among `live` that ended before the step in flight: their token is ignored
            while True:
                # the step after the one whose tokens are still on their way, for every sequence that
                # cannot end at that token for a reason known beforehand
                launched = None
                if ahead and hasattr(picked, "tokens"):
                    rows = [k for k, (i, slot) in enumerate(live)
                            if i not in dropped and len(results[i].tokens) + 1 < sample_len
                            and engine.length(slot) + 1 <= engine.max_context]
                    if rows:
                        logits = engine.step_ahead([live[k][1] for k in rows], rows, picked)
                        if logits is not None:
                            nxt = [live[k] for k in rows]
                            launched = (nxt, sampler.pick_device(logits, [i for i, _ in nxt],
                                                                 [len(results[i].tokens) + 1 for i, _ in nxt]))
                            stats.steps += 1
                tokens = picked.tokens() if hasattr(picked, "tokens") else picked
                survivors = []
                for (i, slot), tok in zip(live, tokens):
                    if i in dropped:
                        continue
                    r = results[i]
                    r.tokens.append(tok)
                    stats.generated_tokens += 1
                    if not from_prompt:
                        stats.decode_tokens += 1
                    if on_token is not None:
                        on_token(i, tok)
                    if tok in stop:
                        r.finish_reason = "stop"
                    elif len(r.tokens) >= sample_len:
                        r.finish_reason = "length"
                    elif engine.length(slot) + (0 if launched and (i, slot) in launched[0] else 1) > engine.max_context:
                        r.finish_reason = "length"
                    if r.finish_reason is None:
                        survivors.append((i, slot))
                    else:
                        close(slot)
                from_prompt = False
                if launched is not None:
                    live, picked = launched
                    dropped = {i for i, _ in live if results[i].finish_reason is not None}
                    if len(dropped) == len(live):
                        break
                    continue
                live, dropped = survivors, set()
                if not live:
                    break
                logits = engine.step([(slot, [results[i].tokens[-1]], [0]) for i, slot in live])
                requests, indices = [i for i, _ in live], [len(results[i].tokens) for i, _ in live]
                picked = sampler.pick_device(logits, requests, indices) if ahead else sampler.pick(logits, requests, indices)
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
