"""The bfloat16 engine against the plain implementation *with the engine's roundings*.

Against the exact plain implementation a bfloat16 run differs by 1.5-3 % of the largest logit, which
is what rounding the activations to 8 bits costs; a fault that only the bfloat16 kernels have and
that moves logits by a percent hides in that.  Here the plain implementation rounds where the
engine rounds (``plain_llama.Rounding``), so that what is left is the order of float32 sums and,
now and then, a value that sits so close to the middle between two bfloat16 neighbours that the
two computations round it to different sides; such a flip moves a row of logits by up to some
tenths of a percent in a model this small; and once it has happened in a key or a value, every
later row of the sequence sees it.  So a share of the rows agrees to 1e-5 (all of them until the
first flip of a sequence) and the rest to some 1e-3, and both are asserted: the share of rows that
agree to 1e-5, which a kernel that computes anything else than the modelled function anywhere would
bring to nothing, and the largest difference, which is half to a third of what the exact plain
implementation leaves room for.

Which of the optional roundings apply depends on how many rows a step has, because the engine fuses
more into one kernel when the rows are few; the table below says so per configuration and is part
of what this test pins (it names what each kernel path keeps unrounded)."""
import numpy as np
import pytest

import plain_llama as P
from helpers import TINIES, make_folder, random_tokens, rel_err

pytestmark = pytest.mark.gpu

# (q/k rounded before the rotation, gate/up rounded before the gating, output projection rounded, down
#  projection rounded) for steps of up to 16 rows, of up to 32, of up to 64, of up to 128, of up to 256, and beyond; then
#  whether the attention rounds its probabilities (the matrix-core kernels do, the generic one, which takes
#  head sizes that are no multiple of 16, does not).
#  A: width 64.  Few rows: projection, rotation and cache write are one kernel, the gating is the
#     product's epilogue.  Up to 256 rows projection, rotation and cache write stay one kernel (these
#     models have few columns); beyond, every product is the library's and is rounded.
#  B: head size 24: up to 16 rows the rotation is a kernel of its own, so q and k are rounded before it; from
#     17 to 256 rows projection, rotation and cache write are one kernel again (the one that takes any even
#     head size).
#  C: width 512, inner 1408: with few rows the down projection comes as unrounded partial sums over
#     two halves of its long inner dimension, and so it does from 65 to 256 rows; from 129 rows on the
#     gate/up product is the fused matrix-core kernel again (its tiles then fill enough of the chip).
STYLES = {
    "A": (((False, False, True, True), (False, False, True, True), (False, False, True, True), (False, True, True, True),
           (False, True, True, True), (True, True, True, True)), True),
    "B": (((True, False, True, True), (False, False, True, True), (False, False, True, True), (False, True, True, True),
           (False, True, True, True), (True, True, True, True)), False),
    "C": (((False, False, True, False), (False, False, True, False), (False, False, True, False), (False, True, True, False),
           (False, False, True, False), (True, False, True, True)), True),
}
LENGTHS = [1, 2, 7, 16, 33, 64, 65, 100, 150, 300]
# least share of rows that agree to 1e-5, and largest row error allowed (of the row's largest logit)
LIMITS = {"A": (0.5, 1.2e-2), "B": (0.1, 1.5e-2), "C": (0.0, 1.5e-2)}


def style_for(name, rows):
    styles, _ = STYLES[name]
    return styles[0 if rows <= 16 else 1 if rows <= 32 else 2 if rows <= 64 else 3 if rows <= 128 else 4 if rows <= 256 else 5]


def rounding_for(name, step_rows_of_token, decoded):
    """One flag per token from the size of the step that fed it; decoded: which tokens came one by one."""
    per_token = np.array([style_for(name, r) for r in step_rows_of_token])
    flags = [per_token[:, k] for k in range(4)]
    return P.Rounding(*flags, probabilities=STYLES[name][1], probability_pages=64, running_maximum=~decoded)


@pytest.fixture(scope="module", params=["A", "B", "C"])
def case(request, tmp_path_factory):
    from burn_lm_amd.engine.loading import load_engine
    cfg, seed = TINIES[request.param]
    folder = make_folder(tmp_path_factory.mktemp("model" + request.param), cfg, seed)
    plain = P.load_model_folder(folder)
    eng = load_engine(folder, dtype="bfloat16", max_tokens=4096)
    reqs = [random_tokens(300 * seed + i, cfg["vocab_size"], n) for i, n in enumerate(LENGTHS)]
    return request.param, eng, plain, reqs


def check(name, errors):
    errors = np.asarray(errors)
    exact, worst = float((errors <= 1e-5).mean()), float(errors.max())
    print(f"config {name}: {errors.size} rows, {exact:.0%} agree to 1e-5, median {np.median(errors):.2e}, "
          f"99 % {np.quantile(errors, 0.99):.2e}, largest {worst:.2e}")
    assert exact >= LIMITS[name][0] and worst <= LIMITS[name][1], (exact, worst)


def test_whole_prompts_against_the_plain_implementation_with_the_engines_roundings(case):
    name, eng, plain, reqs = case
    errors = []
    for t in reqs:
        n = len(t)
        s = eng.open()
        got = eng.step([(s, t, list(range(n)))]).double().cpu().numpy()
        eng.close(s)
        want = P.transformer_forward([t], plain, rounding=rounding_for(name, [n] * n, np.zeros(n, bool)))[0]
        errors += [rel_err(got[p], want[p]) for p in range(n)]
    check(name, errors)


def test_tokens_one_by_one_against_the_plain_implementation_with_the_engines_roundings(case):
    """The last 32 tokens of each request one by one: they bring the roundings of single-row steps, the
    prefix those of its own step, and both meet in the attention."""
    name, eng, plain, reqs = case
    errors = []
    for t in reqs:
        n = len(t)
        head = max(0, n - 32)
        s = eng.open()
        rows = []
        if head:
            rows.append(eng.step([(s, t[:head], list(range(head)))]).double().cpu().numpy())
        for p in range(head, n):
            rows.append(eng.step([(s, [t[p]], [0])]).double().cpu().numpy())
        eng.close(s)
        got = np.concatenate(rows)
        decoded = np.arange(n) >= head
        want = P.transformer_forward([t], plain, rounding=rounding_for(name, np.where(decoded, 1, head), decoded))[0]
        errors += [rel_err(got[p], want[p]) for p in range(n)]
    check(name, errors)
