"""Trace replay through bin/trace_run, as a user runs it, against the plain implementation:
each request whole; with its last 32 tokens one by one; and in batches of unequal lengths whose
shorter requests end earlier, one batch after another on a cache so small that pages and slots
are used again.  In 32-bit and in bfloat16, on two tiny configurations and a middle-sized one."""
import numpy as np
import pytest

import plain_llama as P
from helpers import TINIES, TOL, Trace, make_folder, random_tokens, rel_err, run_trace
from test_bf16_roundings import rounding_for

pytestmark = pytest.mark.gpu

LENGTHS = [1, 2, 33, 64, 65, 100, 7, 150]


@pytest.fixture(scope="module", params=["A", "B", "C"])
def case(request, tmp_path_factory):
    cfg, seed = TINIES[request.param]
    folder = make_folder(tmp_path_factory.mktemp("model" + request.param), cfg, seed)
    plain = P.load_model_folder(folder)
    reqs = {f"r{i}": random_tokens(100 * seed + i, cfg["vocab_size"], n) for i, n in enumerate(LENGTHS)}
    want = {rid: P.transformer_forward([t], plain)[0] for rid, t in reqs.items()}
    return request.param, folder, reqs, want, plain


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
    name, folder, reqs, want, plain = case
    tr, mode_of = build_trace(reqs)
    out = run_trace(folder, dtype, tr, tmp_path / "out")
    worst = {"whole": 0.0, "tail": 0.0, "batched": 0.0}
    seen = {m: set() for m in worst}
    rounded, excused = {}, 0
    for step, rows in tr.index.items():
        got = out[step]
        for k, (rid, pos) in enumerate(rows):
            e = rel_err(got[k], want[rid][pos])
            m = mode_of[step]
            seen[m].add((rid, pos))
            if e > TOL[dtype] and dtype == "bfloat16":
                # About one row in a thousand of configuration B sits on a near-tie of its attention: exact
                # arithmetic between the engine's roundings (the plain implementation with roundings, on the
                # CPU) is then 0.03-0.04 of the largest logit from the exact result by itself (request r5, row
                # 89: 0.042).  Such a row has to agree with that computation instead, and twice as closely.
                fed = tr.history[step, rid]
                if (step, rid) not in rounded:
                    style = rounding_for(name, np.array([r for r, _ in fed]), np.array([d for _, d in fed]))
                    rounded[step, rid] = P.transformer_forward([reqs[rid][:len(fed)]], plain, rounding=style)[0]
                by_rounding = rel_err(rounded[step, rid][pos], want[rid][pos])
                assert by_rounding > 0.8 * TOL[dtype] and rel_err(got[k], rounded[step, rid][pos]) <= TOL[dtype] / 2, \
                    (f"config {name} {m}: request {rid} position {pos} differs by {e:.3g}; roundings alone give {by_rounding:.3g}")
                excused += 1
                continue
            if e > worst[m]:
                worst[m] = e
            assert e <= TOL[dtype], (f"config {name} {dtype} {m}: request {rid} position {pos} of "
                                     f"{len(reqs[rid])} (step {step}) differs by {e:.3g} of the largest logit")
    assert excused <= 3, excused
    everything = {(rid, p) for rid, t in reqs.items() for p in range(len(t))}
    assert seen["whole"] == everything and seen["tail"] == everything
    assert len(seen["batched"]) > 400
    print(f"config {name} {dtype}: worst relative error {worst}")


def test_cache_is_sized_by_max_tokens(case, tmp_path):
    """--max-tokens counts each live request rounded up to 64: one token too few pages must be
    refused by the cache, not answered wrongly."""
    name, folder, reqs, _, _ = case
    tr = Trace()
    tr.step([("a", 0, reqs["r5"][:65], [64]), ("b", 0, reqs["r2"], [0])])   # 128 + 64 tokens of room
    assert tr.peak == 192
    out = run_trace(folder, "float32", tr, tmp_path / "ok", max_tokens=192)
    assert out[0].shape[0] == 2
    with pytest.raises(AssertionError, match="pages"):
        run_trace(folder, "float32", tr, tmp_path / "short", max_tokens=128)


# ---- many concurrent requests ------------------------------------------------------------------

@pytest.fixture(scope="module")
def crowd(tmp_path_factory):
    """Config C and 70 requests of unequal lengths with the plain logits of every position that a
    crowd trace asks for (the last four places of each prefix and every decoded token)."""
    cfg, seed = TINIES["C"]
    folder = make_folder(tmp_path_factory.mktemp("crowdC"), cfg, seed)
    plain = P.load_model_folder(folder)
    lengths = [3 + (37 * i + 11 * (i % 7)) % 118 for i in range(70)]
    reqs = {f"c{i}": random_tokens(5000 + i, cfg["vocab_size"], n) for i, n in enumerate(lengths)}
    want = {rid: P.transformer_forward([t], plain)[0] for rid, t in reqs.items()}
    return folder, reqs, want


def crowd_trace(reqs):
    """Batches of 20, 40 and 70 requests that start together, each batch run twice with other shares
    of prefilled and decoded tokens, one batch after another on a cache that holds one batch: the
    decode steps have 17 to 64 and more than 64 live sequences until the shorter ones have ended."""
    tr = Trace()
    ids = list(reqs)
    for n, first in ((20, 0), (40, 20), (70, 0)):
        for turn in (0, 1):
            batch = ids[first:first + n]
            entries, left = [], {}
            for k, rid in enumerate(batch):
                toks = reqs[rid]
                d = min(len(toks) - 1, (5 * k + 3 * turn) % 14 + (3 if n == 70 else 0))   # tokens decoded one by one
                p = len(toks) - d
                entries.append((rid, 0, toks[:p], list(range(max(0, p - 4), p))))
                left[rid] = p
            tr.step(entries, end=[rid for rid, p in left.items() if p == len(reqs[rid])])
            left = {rid: p for rid, p in left.items() if p < len(reqs[rid])}
            while left:
                entries = [(rid, p, [reqs[rid][p]], [0]) for rid, p in left.items()]
                ending = [rid for rid, p in left.items() if p + 1 == len(reqs[rid])]
                tr.step(entries, end=ending)
                left = {rid: p + 1 for rid, p in left.items() if rid not in ending}
    return tr


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_of_twenty_forty_and_seventy_concurrent_requests(crowd, dtype, tmp_path):
    folder, reqs, want = crowd
    tr = crowd_trace(reqs)
    out = run_trace(folder, dtype, tr, tmp_path / "out")
    worst, rows_checked, widest = 0.0, 0, 0
    for step, rows in tr.index.items():
        got = out[step]
        widest = max(widest, len({rid for rid, _ in rows}))
        for k, (rid, pos) in enumerate(rows):
            e = rel_err(got[k], want[rid][pos])
            worst = max(worst, e)
            rows_checked += 1
            assert e <= TOL[dtype], (f"{dtype}: request {rid} position {pos} of {len(reqs[rid])} (step {step}, "
                                     f"{len(rows)} rows) differs by {e:.3g} of the largest logit")
    assert widest == 70 and rows_checked > 2000
    print(f"crowd {dtype}: {rows_checked} rows, worst relative error {worst:.3g}")
