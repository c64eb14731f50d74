"""The generation loop's decisions, on a stand-in engine without a GPU: batches of unequal
prompts, stop tokens, sequences that end earlier, one batch after another on the same slots."""
import pytest
import torch

from burn_lm_amd.cache.cache import Cache
from burn_lm_amd.engine.generate import generate, plan_batches
from burn_lm_amd.parts.base import KVNeed
from burn_lm_amd.sampling.sampler import Sampler, uniform


class ToyEngine:
    """Next token = (sum of the sequence so far) mod vocab, told through one-hot logits.  Uses the
    real cache bookkeeping, and records every step it is asked to run."""

    def __init__(self, vocab=50, max_tokens=256, max_seqs=4, max_context=64, page=16):
        self.vocab_size, self.max_context = vocab, max_context
        self.cache = Cache([KVNeed(1, 2)], [None], max_tokens, max_seqs, max_context, page, torch.float32, "cpu")
        self.sums, self.steps, self.opened = {}, [], []

    def open(self):
        s = self.cache.open()
        self.sums[s] = 0
        self.opened.append(s)
        return s

    def close(self, s):
        self.cache.close(s)
        del self.sums[s]

    def length(self, s):
        return self.cache.length(s)

    def step(self, entries):
        self.cache.reserve([(s, len(t)) for s, t, _ in entries])
        self.steps.append([(s, len(t)) for s, t, _ in entries])
        rows = []
        for s, toks, want in entries:
            assert want in ([len(toks) - 1], [])    # a prompt's earlier pieces ask for nothing
            self.sums[s] += sum(toks)
            self.cache.advance(s, len(toks))
            if want:
                row = torch.zeros(self.vocab_size)
                row[self.sums[s] % self.vocab_size] = 1.0
                rows.append(row)
        return torch.stack(rows) if rows else None


class HostArgmax:
    def pick(self, logits, requests, indices):
        self.last = (list(requests), list(indices))
        return [int(i) for i in logits.argmax(1)]


def expected(prompt, n, vocab=50, stop=()):
    toks, out = list(prompt), []
    for _ in range(n):
        t = sum(toks) % vocab
        out.append(t); toks.append(t)
        if t in stop:
            break
    return out


def test_unequal_prompts_one_prefill_then_one_token_each():
    eng = ToyEngine()
    prompts = [[1, 2, 3], [4] * 9, [7]]
    res, stats = generate(eng, prompts, HostArgmax(), sample_len=5, batch_size=4)
    assert [r.tokens for r in res] == [expected(p, 5) for p in prompts]
    assert all(r.finish_reason == "length" for r in res)
    assert [n for _, n in eng.steps[0]] == [3, 9, 1]                 # all prompts in one step
    assert all(n == 1 for st in eng.steps[1:] for _, n in st)        # then one token each
    assert len(eng.steps) == 5                                       # the 5th token needs no further step
    assert stats.prompt_tokens == 13 and stats.generated_tokens == 15 and stats.decode_tokens == 12
    assert eng.cache.pages_in_use() == 0 and eng.cache.free_slots == 4


def test_stop_token_ends_a_sequence_and_the_others_go_on():
    eng = ToyEngine()
    prompts = [[1, 2, 3], [5, 5], [9]]
    free = [expected(p, 8) for p in prompts]
    stop = free[1][2]                       # third token of request 1
    want = [expected(p, 8, stop=(stop,)) for p in prompts]
    res, _ = generate(eng, prompts, HostArgmax(), sample_len=8, stop_ids=[stop], batch_size=4)
    assert [r.tokens for r in res] == want
    assert res[1].finish_reason == "stop" and res[1].tokens[-1] == stop and len(res[1].tokens) == 3
    sizes = [len(s) for s in eng.steps]
    assert sizes[0] == 3 and min(sizes) < 3, "the ended sequence must leave the batch"
    # no step runs for a sequence after its stop token
    slot1 = eng.opened[1]
    assert sum(1 for st in eng.steps for s, _ in st if s == slot1) == 3


def test_batches_run_one_after_another_on_the_same_slots():
    eng = ToyEngine(max_seqs=2)
    prompts = [[i + 1] * (i + 1) for i in range(5)]
    res, _ = generate(eng, prompts, HostArgmax(), sample_len=3, batch_size=2)
    assert [r.tokens for r in res] == [expected(p, 3) for p in prompts]
    assert len(eng.opened) == 5 and set(eng.opened) == {0, 1}, "slots are used again"
    assert [len(s) for s in eng.steps if s[0][1] > 1 or len(s) == 2][:1] == [2]
    assert eng.cache.pages_in_use() == 0


def test_batches_are_cut_to_what_the_cache_holds():
    # 4 pages of 16: each request may reach 10 + 20 = 30 tokens = 2 pages -> two per batch
    assert plan_batches([10, 10, 10], 20, batch_size=8, max_context=64, page_size=16, n_pages=4, n_slots=8) == [[0, 1], [2]]
    assert plan_batches([10] * 5, 20, batch_size=2, max_context=64, page_size=16, n_pages=64, n_slots=8) == [[0, 1], [2, 3], [4]]
    assert plan_batches([10] * 3, 20, batch_size=8, max_context=64, page_size=16, n_pages=64, n_slots=1) == [[0], [1], [2]]
    # the context bounds what a request can come to hold
    assert plan_batches([10, 10], 1000, batch_size=8, max_context=32, page_size=16, n_pages=4, n_slots=8) == [[0, 1]]
    eng = ToyEngine(max_tokens=64)
    res, _ = generate(eng, [[1] * 10, [2] * 10, [3] * 10], HostArgmax(), sample_len=20, batch_size=8)
    assert [len(r.tokens) for r in res] == [20, 20, 20]
    assert [len(s) for s in eng.steps if s[0][1] == 10] == [2, 1]


def test_context_end_and_refused_prompts():
    eng = ToyEngine(max_context=12, max_tokens=64)
    res, _ = generate(eng, [[1] * 10, [2] * 13, [], [3]], HostArgmax(), sample_len=50, batch_size=4)
    # 10 prompt tokens + 2 fed-back tokens fill the context; the token predicted from the full context is the last
    assert res[0].finish_reason == "length" and len(res[0].tokens) == 3
    assert res[0].tokens == expected([1] * 10, 3)
    assert res[1].finish_reason == "error" and "exceeds maximum context window (12" in res[1].error
    assert res[2].finish_reason == "error" and not res[2].tokens
    assert res[3].finish_reason == "length" and len(res[3].tokens) == 12
    assert eng.cache.pages_in_use() == 0


def test_a_batch_of_long_prompts_is_fed_in_steps_of_the_budget():
    """Prompts of 5, 3, 9 and 1 tokens with a budget of 6: three steps, the sequences in order, a prompt
    cut where a step is full, logits asked for with each prompt's last piece only; tokens and statistics
    as with one step."""
    from burn_lm_amd.engine.generate import plan_prompt_steps
    assert plan_prompt_steps([5, 3, 9, 1], 6) == [[(0, 0, 5), (1, 0, 1)], [(1, 1, 2), (2, 0, 4)], [(2, 4, 5), (3, 0, 1)]]
    assert plan_prompt_steps([5, 3], 8) == [[(0, 0, 5), (1, 0, 3)]]
    assert plan_prompt_steps([13], 4) == [[(0, 0, 4)], [(0, 4, 4)], [(0, 8, 4)], [(0, 12, 1)]]
    assert plan_prompt_steps([], 4) == []
    with pytest.raises(ValueError):
        plan_prompt_steps([3, 0], 4)
    prompts = [[1, 2, 3, 4, 5], [4] * 3, [7, 1, 2, 3, 4, 5, 6, 7, 8], [9]]
    whole_eng = ToyEngine(max_tokens=512)
    whole, whole_stats = generate(whole_eng, prompts, HostArgmax(), sample_len=5, batch_size=4)
    eng = ToyEngine(max_tokens=512)
    res, stats = generate(eng, prompts, HostArgmax(), sample_len=5, batch_size=4, prompt_budget=6)
    assert [r.tokens for r in res] == [r.tokens for r in whole] == [expected(p, 5) for p in prompts]
    s = eng.opened
    assert eng.steps[:3] == [[(s[0], 5), (s[1], 1)], [(s[1], 2), (s[2], 4)], [(s[2], 5), (s[3], 1)]]
    assert all(n == 1 for st in eng.steps[3:] for _, n in st) and len(eng.steps[3]) == 4
    assert stats.prompt_tokens == whole_stats.prompt_tokens == 18
    assert stats.steps == whole_stats.steps + 2 and stats.generated_tokens == whole_stats.generated_tokens
    assert eng.cache.pages_in_use() == 0 and eng.cache.free_slots == 4
    # a budget that the prompts do not exceed changes nothing
    eng2 = ToyEngine(max_tokens=512)
    generate(eng2, prompts, HostArgmax(), sample_len=5, batch_size=4, prompt_budget=18)
    assert eng2.steps == whole_eng.steps
    with pytest.raises(ValueError):
        generate(eng, prompts, HostArgmax(), sample_len=5, prompt_budget=0)


def test_a_request_that_cannot_fit_the_cache_ends_with_an_error_and_the_others_run():
    # pages of 16 and 4 of them; a context of 128: the second request may grow to 100 tokens = 7 pages
    unfit = []
    assert plan_batches([10, 90, 10], 10, 8, 128, 16, 4, 8, unfit) == [[0, 2]] and unfit == [1]
    eng = ToyEngine(max_tokens=64, max_context=64)
    eng.max_context = 128       # an engine whose context is longer than its cache (several groups of layers can make it so)
    res, _ = generate(eng, [[1] * 10, [2] * 90, [3] * 10], HostArgmax(), sample_len=10, batch_size=8)
    assert res[1].finish_reason == "error" and "pages" in res[1].error and not res[1].tokens
    assert [r.tokens for r in (res[0], res[2])] == [expected([1] * 10, 10), expected([3] * 10, 10)]
    assert eng.cache.pages_in_use() == 0 and eng.cache.free_slots == 4


def test_a_prompt_step_that_the_cache_refuses_fails_its_request_only():
    """The planner counts pages; a cache may still refuse (here: a stand-in that takes no more than 30 new tokens
    per step).  The batch is tried again one request at a time, the one that is refused alone ends with
    the cache's message, nothing stays open."""
    from burn_lm_amd.cache.cache import CacheFull

    class Narrow(ToyEngine):
        def step(self, entries):
            if sum(len(t) for _, t, _ in entries) > 30:
                raise CacheFull("no room for %d tokens" % sum(len(t) for _, t, _ in entries))
            return super().step(entries)

    eng = Narrow(max_tokens=256)
    prompts = [[1] * 10, [2] * 40, [3] * 12]
    res, _ = generate(eng, prompts, HostArgmax(), sample_len=4, batch_size=4)
    assert res[1].finish_reason == "error" and "no room for 40" in res[1].error
    assert [r.tokens for r in (res[0], res[2])] == [expected(prompts[0], 4), expected(prompts[2], 4)]
    assert [r.finish_reason for r in (res[0], res[2])] == ["length", "length"]
    assert eng.cache.pages_in_use() == 0 and eng.cache.free_slots == 4


def test_sample_len_zero_and_callback_order():
    eng = ToyEngine()
    res, _ = generate(eng, [[1, 2]], HostArgmax(), sample_len=0)
    assert res[0].tokens == [] and res[0].finish_reason == "length" and not eng.steps
    seen = []
    res, _ = generate(eng, [[1, 2], [3]], HostArgmax(), sample_len=3, on_token=lambda r, t: seen.append((r, t)))
    assert [t for r, t in seen if r == 0] == res[0].tokens and [t for r, t in seen if r == 1] == res[1].tokens
    assert [r for r, _ in seen[:2]] == [0, 1]


def test_slots_are_returned_when_a_step_fails():
    eng = ToyEngine()

    def boom(entries):
        raise RuntimeError("kernel failed")
    eng.step = boom
    with pytest.raises(RuntimeError, match="kernel failed"):
        generate(eng, [[1], [2]], HostArgmax(), sample_len=2)
    assert eng.cache.free_slots == 4


def test_sampler_numbers_depend_on_seed_request_and_index_only():
    a = Sampler(0.8, 0.9, seed=5)
    assert a.uniforms([3, 4], [0, 0]) == [uniform(5, 3, 0), uniform(5, 4, 0)]
    assert a.uniforms([3], [7]) == a.uniforms([9, 3], [1, 7])[1:]       # batch mates do not matter
    assert uniform(5, 3, 0) != uniform(6, 3, 0) != uniform(5, 3, 1)
    us = [uniform(1, r, i) for r in range(40) for i in range(50)]
    assert all(0.0 <= u < 1.0 for u in us) and abs(sum(us) / len(us) - 0.5) < 0.02
    assert Sampler(0.0).greedy and not a.greedy
    assert Sampler(0.7, seed=0).seed != Sampler(0.7, seed=0).seed       # 0 = a fresh seed each time
    with pytest.raises(ValueError):
        Sampler(-1.0)
    with pytest.raises(ValueError):
        Sampler(1.0, top_p=0.0)


def test_sampler_is_told_request_and_token_index():
    eng = ToyEngine()
    s = HostArgmax()
    generate(eng, [[1], [20], [3]], s, sample_len=4, stop_ids=[expected([20], 4)[1]], batch_size=4)
    assert s.last == ([0, 2], [3, 3])


class AheadEngine(ToyEngine):
    """A stand-in with step_ahead: a shape (number of sequences) can run ahead once a plain decode
    step of that shape has run, as a recorded graph would allow."""

    def __init__(self, **kw):
        super().__init__(**kw)
        self.recorded, self.ahead_steps = set(), 0

    def step(self, entries):
        if all(len(t) == 1 for _, t, _ in entries):
            self.recorded.add(len(entries))
        return super().step(entries)

    def step_ahead(self, slots, rows, picked):
        if len(slots) not in self.recorded:
            return None
        self.ahead_steps += 1
        toks = picked.tokens()      # the stand-in may look; the real engine takes them on the device
        return super().step([(s, [toks[r]], [0]) for s, r in zip(slots, rows)])


class ToyPicked:
    def __init__(self, toks):
        self._toks = toks
        self.read = False

    def tokens(self):
        self.read = True
        return list(self._toks)


class AheadArgmax(HostArgmax):
    def pick_device(self, logits, requests, indices):
        self.calls = getattr(self, "calls", []) + [(list(requests), list(indices))]
        return ToyPicked(self.pick(logits, requests, indices))


def test_running_ahead_gives_the_same_tokens_and_at_most_one_dropped_step_per_stop():
    prompts = [[1, 2, 3], [5, 5], [9], [2, 7, 1, 1]]
    free = [expected(p, 9) for p in prompts]
    stop = free[1][2]
    want = [expected(p, 9, stop=(stop,)) for p in prompts]
    plain_eng = ToyEngine()
    plain, _ = generate(plain_eng, prompts, HostArgmax(), sample_len=9, stop_ids=[stop], batch_size=4)
    eng, sampler = AheadEngine(), AheadArgmax()
    res, stats = generate(eng, prompts, sampler, sample_len=9, stop_ids=[stop], batch_size=4)
    assert [r.tokens for r in res] == want == [r.tokens for r in plain]
    assert [r.finish_reason for r in res] == [r.finish_reason for r in plain]
    assert eng.ahead_steps > 0, "no step ran ahead"
    # a sequence that met its stop token was in one more step than without running ahead; one that
    # ended at sample_len was not
    def steps_of(e, k):
        return sum(1 for st in e.steps for s, _ in st if s == e.opened[k])
    for k, r in enumerate(res):
        extra = steps_of(eng, k) - steps_of(plain_eng, k)
        assert extra == (1 if r.finish_reason == "stop" else 0), (k, r.finish_reason, extra)
    assert stats.generated_tokens == sum(len(w) for w in want)
    assert stats.decode_tokens == stats.generated_tokens - len(prompts)
    # the random number of a draw is that of the token's index in its request, also when picked ahead
    for requests, indices in sampler.calls:
        assert len(requests) == len(indices)
    assert eng.cache.pages_in_use() == 0 and eng.cache.free_slots == 4


def test_running_ahead_stops_at_the_end_of_the_context_without_an_extra_step():
    eng = AheadEngine(max_context=12, max_tokens=64)
    res, _ = generate(eng, [[1] * 10, [3]], AheadArgmax(), sample_len=50, batch_size=4)
    assert res[0].finish_reason == "length" and res[0].tokens == expected([1] * 10, 3)
    assert res[1].finish_reason == "length" and len(res[1].tokens) == 12
    assert eng.cache.pages_in_use() == 0
    assert max(n for st in eng.steps for _, n in st if n == 1) == 1
    for s in eng.opened:
        assert s not in eng.cache.live_slots


def test_the_native_core_draws_the_same_uniforms_and_plans_the_same_batches():
    """The host core (C++) holds the loop's decisions; its random numbers are the function `uniform`."""
    import ctypes
    from burn_lm_amd.cache import core
    from burn_lm_amd.engine.generate import plan_batches
    reqs, idx = [0, 3, 7, 100, 2 ** 20], [0, 1, 5000, 3, 9]
    out = (ctypes.c_float * 5)()
    core.library().blm_uniforms(12345678901234567, 5, core.ints(reqs), core.ints(idx), ctypes.cast(out, ctypes.c_void_p))
    assert list(out) == [uniform(12345678901234567, r, i) for r, i in zip(reqs, idx)]
    # batches: at most 3 sequences, and pages for prompt + sample_len each (pages of 64, 10 pages in all)
    assert plan_batches([5, 200, 70, 1, 300, 9], 60, 3, 1024, 64, 10, 8) == [[0, 1, 2], [3, 4, 5]]   # 2 + 5 + 3 pages, then 1 + 6 + 2
    assert plan_batches([5, 200, 70, 1, 300, 9], 60, 3, 1024, 64, 9, 8) == [[0, 1], [2, 3], [4, 5]]      # one page fewer
    assert plan_batches([5, 5, 5, 5], 10, 3, 1024, 64, 100, 2) == [[0, 1], [2, 3]]      # two slots only
    assert plan_batches([], 10, 3, 1024, 64, 100, 2) == []


def test_the_native_core_decides_which_steps_are_replayed():
    """blm_step_key: the bucket of a step that wants each sequence's last token only; -1 otherwise."""
    import ctypes
    from burn_lm_amd.cache import core
    from burn_lm_amd.engine import graphs

    def key(counts, lengths, wants):
        p = core.Packed([(i, [0] * c, w) for i, (c, w) in enumerate(zip(counts, wants))])
        k = (ctypes.c_int * 3)()
        core.library().blm_step_key(p.n, p.counts, core.ints(lengths), p.want_counts, p.wants, len(graphs.BATCH_BUCKETS),
                                    graphs._BATCH_BUCKETS, len(graphs.TOKEN_BUCKETS), graphs._TOKEN_BUCKETS,
                                    graphs.PROMPT_MAX_SEQS, 64, 64, k)
        return tuple(k) if k[0] >= 0 else None

    assert key([1, 1, 1], [10, 700, 3], [[0], [0], [0]]) == (4, 0, 16)          # decode: 3 -> bucket 4, 11 pages -> 16
    assert key([1], [5], [[0]]) == (1, 0, 8)
    assert key([40, 7, 90], [0, 0, 0], [[39], [6], [89]]) == (4, 256, 8)        # prompts: 137 tokens -> 256
    assert key([40, 7], [0, 0], [[39], [5]]) is None                            # not the last token
    assert key([40, 7], [0, 0], [[39], []]) is None                             # nothing wanted
    assert key([3000], [0], [[2999]]) is None                                   # beyond the token buckets
    assert key([2] * 17, [0] * 17, [[1]] * 17) is None                          # too many sequences for a prompt step
    assert key([1] * 129, [0] * 129, [[0]] * 129) is None                       # beyond the batch buckets
    assert key([1], [64 * 64 - 1], [[0]]) == (1, 0, 64)                         # the widest table
