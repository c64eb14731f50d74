"""Trace replay through bin/trace_run, as a user runs it, against the plain implementation:
each request whole; with its last 32 tokens one by one; and in batches of unequal lengths whose
shorter requests end earlier, one batch after another on a cache so small that pages and slots
are used again.  In 32-bit and in bfloat16, on two tiny configurations and a middle-sized one."""
import pytest

import plain_llama as P
from helpers import TINIES, TOL, Trace, make_folder, random_tokens, rel_err, run_trace

pytestmark = pytest.mark.gpu

LENGTHS = [1, 2, 33, 64, 65, 100, 7, 150]


@pytest.fixture(scope="module", params=["A", "B", "C"])
def case(request, tmp_path_factory):
    cfg, seed = TINIES[request.param]
    folder = make_folder(tmp_path_factory.mktemp("model" + request.param), cfg, seed)
    plain = P.load_model_folder(folder)
    reqs = {f"r{i}": random_tokens(100 * seed + i, cfg["vocab_size"], n) for i, n in enumerate(LENGTHS)}
    want = {rid: P.transformer_forward([t], plain)[0] for rid, t in reqs.items()}
    return request.param, folder, reqs, want


def build_trace(reqs):
    tr = Trace()
    mode_of = {}
    # 1. each request alone and whole, every position wanted
    for rid, toks in reqs.items():
        mode_of[tr.n] = "whole"
        tr.step([(rid, 0, toks, list(range(len(toks))))], end=[rid])
    # 2. each request alone, the last 32 tokens one by one
    for rid, toks in reqs.items():
        head = max(0, len(toks) - 32)
        if head:
            mode_of[tr.n] = "tail"
            tr.step([(rid, 0, toks[:head], list(range(head)))])
        for p in range(head, len(toks)):
            mode_of[tr.n] = "tail"
            tr.step([(rid, p, [toks[p]], [0])], end=[rid] if p == len(toks) - 1 else [])
    # 3. batches of unequal lengths; request i is prefilled up to its last d_i tokens, which are then
    #    decoded one per step, so requests end at different steps; the second and third batch start
    #    after the first has ended and get its slots and pages
    ids = list(reqs)
    for batch, decodes in (([0, 2, 3, 6], [0, 5, 17, 3]), ([1, 4, 5], [1, 30, 9]), ([7, 6, 2, 0], [40, 6, 32, 0])):
        entries, left = [], {}
        for i, d in zip(batch, decodes):
            rid, toks = ids[i], reqs[ids[i]]
            d = min(d, len(toks) - 1)
            p = len(toks) - d
            entries.append((rid, 0, toks[:p], list(range(p))))
            left[rid] = p
        mode_of[tr.n] = "batched"
        tr.step(entries, end=[rid for rid, p in left.items() if p == len(reqs[rid])])
        left = {rid: p for rid, p in left.items() if p < len(reqs[rid])}
        while left:
            entries = [(rid, p, [reqs[rid][p]], [0]) for rid, p in left.items()]
            ending = [rid for rid, p in left.items() if p + 1 == len(reqs[rid])]
            mode_of[tr.n] = "batched"
            tr.step(entries, end=ending)
            left = {rid: p + 1 for rid, p in left.items() if rid not in ending}
    return tr, mode_of


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_matches_plain_whole_tail_and_batched(case, dtype, tmp_path):
    name, folder, reqs, want = case
    tr, mode_of = build_trace(reqs)
    out = run_trace(folder, dtype, tr, tmp_path / "out")
    worst = {"whole": 0.0, "tail": 0.0, "batched": 0.0}
    seen = {m: set() for m in worst}
    for step, rows in tr.index.items():
        got = out[step]
        for k, (rid, pos) in enumerate(rows):
            e = rel_err(got[k], want[rid][pos])
            m = mode_of[step]
            seen[m].add((rid, pos))
            if e > worst[m]:
                worst[m] = e
            assert e <= TOL[dtype], (f"config {name} {dtype} {m}: request {rid} position {pos} of "
                                     f"{len(reqs[rid])} (step {step}) differs by {e:.3g} of the largest logit")
    everything = {(rid, p) for rid, t in reqs.items() for p in range(len(t))}
    assert seen["whole"] == everything and seen["tail"] == everything
    assert len(seen["batched"]) > 400
    print(f"config {name} {dtype}: worst relative error {worst}")


def test_cache_is_sized_by_max_tokens(case, tmp_path):
    """--max-tokens counts each live request rounded up to 64: one token too few pages must be
    refused by the cache, not answered wrongly."""
    name, folder, reqs, _ = case
    tr = Trace()
    tr.step([("a", 0, reqs["r5"][:65], [64]), ("b", 0, reqs["r2"], [0])])   # 128 + 64 tokens of room
    assert tr.peak == 192
    out = run_trace(folder, "float32", tr, tmp_path / "ok", max_tokens=192)
    assert out[0].shape[0] == 2
    with pytest.raises(AssertionError, match="pages"):
        run_trace(folder, "float32", tr, tmp_path / "short", max_tokens=128)
