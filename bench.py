"""Decode and prefill throughput of the engine on one MI355X, with roofline fractions.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 4096] [--layers L]
    python bench.py --preset llama3.2-3b --unequal 16 [--generate 256]     (an unequal batch, end to end)

A "step" is one decode step of the whole batch as the generation loop runs it: the engine's step
function on one token per sequence, the sampling kernel, and the tokens' trip to the host.  Decoding
is measured *through the generation loop itself* (``engine.generate.generate``): prompts that bring
every sequence to the context length, W untimed steps, then exactly K steps between two
synchronisations.  The default run has the layer sizes of the Llama-3.2-1B shape with random weights,
a batch of 8 and a context of 4096 tokens per sequence.  One JSON line is printed:

* ``value``: decoded tokens a second over the K steps; ``ms_per_step`` their mean; ``step_ms_median``
  the median of the single steps (HIP events, one after every step).
* ``roofline``: the bytes a decode step has to read (every weight it uses once and the cache of the
  live requests, as the model's own parts count them) / its time, against 8 TB/s; ``prefill``: a
  prompt of 2,048 tokens through the step function, its flops / time against the dense bf16 peak.
* ``points``: decode at batch 1, 32 and 64 at the same context, with their roofline fractions;
  ``workload_512_256``: the benchmark's second workload (512-token prompts, 256 generated tokens, at
  batch 1, 8 and 64) as decoded tokens a second over the whole decode phase.
* ``measured``: what this machine reaches with a kernel that only reads (GB/s) and one that only
  issues matrix instructions (TFLOP/s), as second denominators; ``kernels``: time and achieved GB/s
  (decode) or TFLOP/s (prefill) of the dominant kernels alone at the benchmark's shape.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0                                   # MI355X HBM3E, published
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}          # dense, published


def random_prompts(engine, n, length, seed=0):
    import numpy as np
    rng = np.random.default_rng(seed)
    return [[int(t) for t in rng.integers(0, engine.vocab_size, length)] for _ in range(n)]


SETTLE_S = float(os.environ.get('BENCH_SETTLE', '0'))


def time_decode(engine, sampler, batch, context, steps, warmup):
    """-> (seconds per step over `steps` steps, median seconds of the single steps).  The batch runs
    through the generation loop: its prompts end `warmup + steps + 2` tokens before the context."""
    import torch
    from burn_lm_amd.engine.generate import generate

    n_new = warmup + steps + 2
    prompts = random_prompts(engine, batch, context - n_new)
    seen, marks, events = [0], {}, []

    def on_token(request, token):
        if request != 0:
            return
        seen[0] += 1        # token 1 comes from the prompt step, token 1 + k from decode step k
        k = seen[0] - 1
        if k == 0 and SETTLE_S > 0:
            torch.cuda.synchronize()
            time.sleep(SETTLE_S)
        if k in (warmup, warmup + steps):
            torch.cuda.synchronize()
            marks[k] = time.perf_counter()
        if warmup <= k <= warmup + steps:
            e = torch.cuda.Event(enable_timing=True)
            e.record()
            events.append(e)

    generate(engine, prompts, sampler, n_new, stop_ids=(), batch_size=batch, on_token=on_token)
    torch.cuda.synchronize()
    singles = [a.elapsed_time(b) * 1e-3 for a, b in zip(events[1:-1], events[2:])]   # the first one follows a synchronisation
    return (marks[warmup + steps] - marks[warmup]) / steps, statistics.median(singles) if singles else float("nan")


def decode_roofline(engine, batch, context, steps, sec):
    mean_ctx = int(context - steps / 2)
    c = engine.model.step_costs([mean_ctx - 1] * batch, [1] * batch, batch, engine.cache)
    achieved = (c["weight_bytes"] + c["cache_bytes"]) / sec / 1e9
    return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4)}


def time_prefill(engine, T, reps=5):
    """Median seconds of a prompt of T tokens through the step function (the first run records nothing: a
    prompt step is replayed from a graph from its second sight on, as in serving)."""
    import torch
    toks = random_prompts(engine, 1, T)[0]
    times = []
    for r in range(reps + 2):
        s = engine.open()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([(s, toks, [T - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        engine.close(s)
        if r >= 2:
            times.append(dt)
    return statistics.median(times)


def time_workload(engine, batch, prompt_len=512, generated=256):
    """The workload of 512-token prompts and 256 generated tokens through the generation loop: decoded tokens a second over the
    decode phase, and prompt tokens a second over the prompt step, of the third of three runs (a shape
    is recorded as a graph the second time it is met, so the third run replays the prompt step too)."""
    from burn_lm_amd.engine.generate import generate
    from burn_lm_amd.sampling.sampler import Sampler
    prompts = random_prompts(engine, batch, prompt_len, seed=1)
    for _ in range(3):
        _, stats = generate(engine, prompts, Sampler(temperature=0.0), generated, stop_ids=(), batch_size=batch)
    return stats.decode_tokens / stats.decode_seconds, stats.prompt_tokens / stats.prompt_seconds


def workload_hbm_frac(engine, batch, steps_per_second, prompt_len=512, generated=256):
    """The 512 + 256 workload's decode steps against the memory roofline: the bytes a step at the
    workload's mean context has to read (every weight once, the live cache) x steps a second / 8 TB/s."""
    mean_ctx = prompt_len + generated // 2
    c = engine.model.step_costs([mean_ctx - 1] * batch, [1] * batch, batch, engine.cache)
    return round((c["weight_bytes"] + c["cache_bytes"]) * steps_per_second / 1e9 / HBM_PEAK_GBS, 4)


def other_shape(name, dtype, batch, context, steps, warmup, prefill_tokens):
    """Decode at `batch` and a prefill of `prefill_tokens` for another preset with all its layers: flat
    figures for the record's `shapes` block."""
    import torch
    from burn_lm_amd.config.presets import preset
    from burn_lm_amd.engine.loading import random_engine
    from burn_lm_amd.sampling.sampler import Sampler
    engine = random_engine(preset(name), seed=0, dtype=dtype, max_tokens=batch * context, max_seqs=batch, max_context=context)
    sec, _ = time_decode(engine, Sampler(temperature=0.0), batch, context, steps, warmup)
    roof = decode_roofline(engine, batch, context, steps, sec)
    psec = time_prefill(engine, prefill_tokens, reps=3)
    pflops = engine.model.step_costs([0], [prefill_tokens], 1)["flops"]
    short = "bf16" if dtype == "bfloat16" else "fp32"
    out = {f"{name}_layers": engine.config.num_hidden_layers,
           f"{name}_decode_b{batch}": round(batch / sec, 1), f"{name}_decode_b{batch}_ms": round(sec * 1e3, 4),
           f"{name}_decode_b{batch}_hbm_frac": roof["frac"],
           f"{name}_prefill_{prefill_tokens}": round(prefill_tokens / psec, 1), f"{name}_prefill_{prefill_tokens}_ms": round(psec * 1e3, 3),
           f"{name}_prefill_{prefill_tokens}_frac": round(pflops / psec / MFMA_PEAK[short], 4)}
    del engine
    torch.cuda.empty_cache()
    return out


def reference_bench_shapes(dtype):
    """The reference's own benchmark (benchmarks/benches/transformer.rs:72-102): one layer of the Llama-3.2-1B, 3B and
    8B shapes with the whole vocabulary, a forward of (batch 32, 1 token) and of (batch 1, 512 tokens) on an empty
    cache with the logits of every position: milliseconds per forward (median)."""
    import torch
    from burn_lm_amd.config.presets import preset
    from burn_lm_amd.engine.loading import random_engine
    out = {}
    for name in ("llama3.2-1b", "llama3.2-3b", "llama3.1-8b"):
        cfg = preset(name)
        cfg["num_hidden_layers"] = 1
        engine = random_engine(cfg, seed=0, dtype=dtype, max_tokens=32 * 64 + 1024, max_seqs=32, max_context=1024)
        for batch, length in ((32, 1), (1, 512)):
            prompts = random_prompts(engine, batch, length, seed=2)
            times = []
            for r in range(8):
                slots = [engine.open() for _ in range(batch)]
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                engine.step([(s, p, list(range(length))) for s, p in zip(slots, prompts)])
                torch.cuda.synchronize()
                times.append(time.perf_counter() - t0)
                for s in slots:
                    engine.close(s)
            out[f"{name}_1layer_b{batch}_s{length}_ms"] = round(statistics.median(times[3:]) * 1e3, 4)
        del engine
        torch.cuda.empty_cache()
    return out


def event_time(fn, reps=10, warm=2):
    """Median seconds of fn() between two events."""
    import torch
    for _ in range(warm):
        fn()
    pairs = []
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        pairs.append((a, b))
    torch.cuda.synchronize()
    return statistics.median(a.elapsed_time(b) for a, b in pairs) * 1e-3


def machine_rates(device):
    import torch
    from burn_lm_amd.csrc import ops
    buf = torch.empty(1 << 30, dtype=torch.uint8, device=device)
    buf.zero_()
    n = ops.probe_read(buf)
    read = n / event_time(lambda: ops.probe_read(buf)) / 1e9
    del buf
    flops = ops.probe_mfma(iters=2048, blocks=2048, device=device)
    mfma = flops / event_time(lambda: ops.probe_mfma(iters=2048, blocks=2048, device=device)) / 1e12
    # the same on random operands that change with every instruction, as a product of real data has them:
    # the clock follows the power the multipliers draw
    rand = flops / event_time(lambda: ops.probe_mfma(iters=2048, blocks=2048, device=device, random_operands=True)) / 1e12
    return {"read_gbs": round(read, 1), "mfma_bf16_tflops": round(mfma, 1), "mfma_bf16_random_tflops": round(rand, 1)}


def kernel_rates(engine, batch, context, prefill_tokens):
    """The dominant kernels alone, at the shapes of the benchmark's decode step and of its prefill, through
    the parts' own methods (so the kernels are the ones a step runs).  A kernel is timed as a recorded
    graph that runs it many times in a row, every time on other weights (the layers' own and copies
    of them, 768 MB and more in all, so that they come from memory as they do in a step and not from
    the 256 MB last-level cache) or on another layer's cache; the time is what one kernel adds to a
    chain of dependent kernels, as in a step.  Decode: achieved GB/s of the weights (or keys and
    values) a kernel reads once; prefill: achieved TFLOP/s."""
    import torch
    from burn_lm_amd.engine.runtime import LinearWeight
    rt, model = engine.rt, engine.model
    blocks = [(model.blocks[pl.layer], engine.cache.views[i]) for i, pl in enumerate(model.plan.order)]
    out = {}

    def spread(weights, least=768 << 20):
        """The layers' weights of one kind and as many copies as it takes to span `least` bytes."""
        size = sum(w.w.numel() * w.w.element_size() for w in weights)
        all_ = list(weights)
        while size < least:
            for w in weights:
                all_.append(LinearWeight(w.w.clone(), w.packable, w.gated))
            size *= 2
        return all_

    def graph_time(calls):
        """Seconds per call of the calls recorded one after another."""
        for c in calls:     # once outside the recording: a weight's packed copy is made at its first product
            c()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for c in calls:
                c()
        return event_time(g.replay) / len(calls)

    def rate(name, calls, nbytes=None, flops=None):
        sec = graph_time(calls)
        out[name + "_us"] = round(sec * 1e6, 2)     # flat keys: a record may drop what lies deeper
        if nbytes is not None:
            out[name + "_gbs"] = round(nbytes / sec / 1e9, 1)
        if flops is not None:
            out[name + "_tflops"] = round(flops / sec / 1e12, 1)

    width = model.plan.width
    m0, f0, v0 = blocks[0][0].mixer, blocks[0][0].feed_forward, blocks[0][1]
    w_bytes = lambda w: w.w.numel() * w.w.element_size()
    nh, nkv, hd = m0.heads, m0.kv_heads, m0.head_dim
    qkvs, os_ = spread([b.mixer.w_qkv for b, _ in blocks]), spread([b.mixer.w_o for b, _ in blocks])
    gus, downs = spread([b.feed_forward.w_gate_up for b, _ in blocks]), spread([b.feed_forward.w_down for b, _ in blocks])
    # ---- a decode step of `batch` sequences that hold `context - 1` tokens ----
    slots = [engine.open() for _ in range(batch)]
    for s in slots:
        engine.cache.reserve([(s, context)])
        engine.cache.advance(s, context - 1)
    step = engine.build_step([(s, [1], [0]) for s in slots])
    x = torch.randn(batch, width, device=rt.device).to(rt.dtype)
    qkv = m0.project(x, step, v0)
    att = m0.attend(qkv, step, v0)
    act = rt.gated_linear(x, f0.w_gate_up)
    kv_bytes = batch * 2 * nkv * hd * context * v0.k.element_size()
    rate("decode_qkv_rope", [lambda w=w: m0.position.project_encode_store(x, w, step, v0, nh, nkv, hd) for w in qkvs],
         nbytes=w_bytes(m0.w_qkv))
    rate("decode_attention", [lambda b=b, v=v: b.mixer.attend(qkv, step, v) for b, v in blocks * 2], nbytes=kv_bytes)
    rate("decode_o", [lambda w=w: rt.linear(att, w, partials=True) for w in os_], nbytes=w_bytes(m0.w_o))
    rate("decode_gate_up", [lambda w=w: rt.gated_linear(x, w) for w in gus], nbytes=w_bytes(f0.w_gate_up))
    rate("decode_down", [lambda w=w: rt.linear(act, w, partials=True) for w in downs], nbytes=w_bytes(f0.w_down))
    heads = spread([model.head.weight])
    rate("decode_head", [lambda w=w: rt.linear(x, w, out_dtype=torch.float32) for w in heads], nbytes=w_bytes(model.head.weight))
    del heads
    for s in slots:
        engine.close(s)
    # ---- a prompt of `prefill_tokens` tokens ----
    T = prefill_tokens
    s = engine.open()
    engine.cache.reserve([(s, T)])
    step = engine.build_step([(s, [1] * T, [T - 1])])
    x = torch.randn(T, width, device=rt.device).to(rt.dtype)
    qkv = m0.project(x, step, v0)
    att = m0.attend(qkv, step, v0)
    act = rt.gated_linear(x, f0.w_gate_up)
    n = len(blocks)
    rate("prefill_qkv_rope", [lambda w=w: m0.position.project_encode_store(x, w, step, v0, nh, nkv, hd) for w in qkvs[:n]],
         flops=2 * T * m0.w_qkv.w.numel())
    rate("prefill_attention", [lambda b=b, v=v: b.mixer.attend(qkv, step, v) for b, v in blocks], flops=m0.mixing_flops(0, T))
    rate("prefill_o", [lambda w=w: rt.linear(att, w, partials=True) for w in os_[:n]], flops=2 * T * m0.w_o.w.numel())
    rate("prefill_gate_up", [lambda w=w: rt.gated_linear(x, w) for w in gus[:n]], flops=2 * T * f0.w_gate_up.w.numel())
    rate("prefill_down", [lambda w=w: rt.linear(act, w, partials=True) for w in downs[:n]], flops=2 * T * f0.w_down.w.numel())
    engine.close(s)
    return out


def run_unequal(args):
    """An unequal batch through the generation loop: --unequal N prompts of 64..2048 seeded random
    tokens in one prefill step, then --generate greedy tokens each.  One JSON line of its own."""
    import numpy as np
    import torch
    from burn_lm_amd.config.presets import preset
    from burn_lm_amd.engine.generate import generate
    from burn_lm_amd.engine.loading import random_engine
    from burn_lm_amd.sampling.sampler import Sampler

    rng = np.random.default_rng(0)
    lens = [int(x) for x in rng.integers(64, 2049, args.unequal)]
    context = (max(lens) + args.generate + 63) // 64 * 64
    engine = random_engine(preset(args.preset), seed=0, dtype=args.dtype, max_tokens=args.unequal * context,
                           max_seqs=args.unequal, max_context=context)
    prompts = [[int(t) for t in rng.integers(0, engine.vocab_size, n)] for n in lens]
    best = None
    for _ in range(3):      # the first runs record the graphs of their shapes
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        _, stats = generate(engine, prompts, Sampler(temperature=0.0), args.generate, batch_size=args.unequal)
        torch.cuda.synchronize()
        whole = time.perf_counter() - t0
        if best is None or whole < best[0]:
            best = (whole, stats)
    whole, stats = best
    print(json.dumps({
        "metric": "generation_seconds", "value": round(whole, 4), "unit": "s", "n_gpus": 1, "higher_is_better": False,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (seeded random weights and token ids)",
        "config": {"model": args.preset, "sequences": args.unequal, "prompt_tokens": sum(lens), "shortest": min(lens),
                   "longest": max(lens), "generated_each": args.generate, "sampling": "greedy"},
        "prefill": {"value": round(stats.prompt_tokens / stats.prompt_seconds, 1), "tokens": stats.prompt_tokens,
                    "ms": round(stats.prompt_seconds * 1e3, 2)},
        "decode": {"value": round(stats.decode_tokens / stats.decode_seconds, 1), "tokens": stats.decode_tokens,
                   "ms": round(stats.decode_seconds * 1e3, 2)}}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (both numbers are reported)")
    ap.add_argument("--preset", default="llama3.2-1b")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and batch 64 points, the 512+256 workload, the single kernels "
                                                             "and the other shapes")
    ap.add_argument("--no-shapes", action="store_true", help="skip the other presets' figures and the reference's own benchmark shapes")
    ap.add_argument("--temperature", type=float, default=0.0, help="sample instead of picking greedily (0: greedy)")
    ap.add_argument("--top-p", type=float, default=1.0, help="nucleus mass when sampling")
    ap.add_argument("--unequal", type=int, default=0, metavar="N",
                    help="instead of the decode measurement: N prompts of 64..2048 tokens through the generation loop")
    ap.add_argument("--generate", type=int, default=256, help="tokens generated per prompt with --unequal")
    ap.add_argument("--profile", choices=["decode", "prefill", "decode-loop"], default=None,
                    help="run only this part, for a profiler: the decode steps of the batch through generate(), the prompt "
                         "step ten times, or (decode-loop, for counter runs, where every launch is slow) --steps decode steps "
                         "launched kernel by kernel on a cache that is filled without a prompt step; prints its time and "
                         "no JSON line, and says on stderr where it is")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this library has no multi-GPU path (run with --gpus 1)")
        sys.exit(2)

    if args.unequal:
        return run_unequal(args)

    from burn_lm_amd.config.presets import preset
    from burn_lm_amd.engine.loading import random_engine
    from burn_lm_amd.sampling.sampler import Sampler

    def say(what):      # a profiled run that stalls should show how far it came
        if args.profile:
            print(f"[bench] {what}", file=sys.stderr, flush=True)

    config = preset(args.preset)
    full_layers = config["num_hidden_layers"]
    layers = args.layers or full_layers
    config["num_hidden_layers"] = layers
    biggest = max(args.batch, 1 if args.no_points else 64)
    from burn_lm_amd.csrc import build as _build
    if args.profile:
        if _build.under_profiler() and not (_build.is_current() and _build.host_is_current()):
            print("bench.py: the kernel libraries do not match their sources; build them before profiling "
                  "(python -c 'import __graft_entry__ as g; g.build()')")
            sys.exit(2)
    # under a profiler every launch is slow (a counter run was seen to take two minutes for the 12,727 small
    # launches of the counter-based weight stream alone): the weights then come from one launch per tensor
    quick = bool(args.profile) and _build.under_profiler()
    say("building the engine (random weights" + (", one launch per tensor)" if quick else ")"))
    engine = random_engine(config, seed=0, dtype=args.dtype, max_tokens=biggest * args.context,
                           max_seqs=biggest, max_context=args.context, graphs=args.profile != "decode-loop",
                           quick_weights=quick)
    say("engine built")
    cfg = engine.config
    page_size = engine.cache.page_size
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    sampler = Sampler(temperature=args.temperature, top_p=args.top_p, seed=1)

    if args.profile == "prefill":
        print(f"prefill of {args.prefill_tokens} tokens: {time_prefill(engine, args.prefill_tokens, reps=10) * 1e3:.3f} ms")
        return
    if args.profile == "decode-loop":
        import torch
        slots = [engine.open() for _ in range(args.batch)]
        for s in slots:     # the cache filled by the books alone: what the pages hold does not matter to the kernels' work
            engine.cache.reserve([(s, args.context - args.steps - 1)])
            engine.cache.advance(s, args.context - args.steps - 1)
        say("cache filled; decode steps, kernel by kernel")
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for k in range(args.steps):
            engine.step([(s, [1 + k], [0]) for s in slots])
        torch.cuda.synchronize()
        print(f"{args.steps} eager decode steps of batch {args.batch} at context {args.context}: "
              f"{(time.perf_counter() - t0) / args.steps * 1e3:.3f} ms each")
        return
    say("decode through generate()")
    sec, median = time_decode(engine, sampler, args.batch, args.context, args.steps, args.warmup)
    if args.profile == "decode":
        print(f"decode step of batch {args.batch} at context {args.context}: {sec * 1e3:.4f} ms")
        return
    value = args.batch / sec

    T = args.prefill_tokens
    psec = time_prefill(engine, T)
    pflops = engine.model.step_costs([0], [T], 1)["flops"]

    points, workload, kernels, measured = {}, {}, {}, {}
    if not args.no_points:
        for b in (1, 32, 64):
            s, _ = time_decode(engine, sampler, b, args.context, max(20, args.steps // 2), 4)
            points[f"decode_b{b}"] = round(b / s, 1)
            points[f"decode_b{b}_ms"] = round(s * 1e3, 4)
            points[f"decode_b{b}_hbm_frac"] = decode_roofline(engine, b, args.context, max(20, args.steps // 2), s)["frac"]
        for b in (1, 8, 64):
            d, p = time_workload(engine, b)
            workload[f"decode_b{b}"] = round(d, 1)
            workload[f"decode_b{b}_hbm_frac"] = workload_hbm_frac(engine, b, d / b)
            workload[f"prefill_b{b}"] = round(p, 1)
        measured = machine_rates(engine.rt.device)
        kernels = kernel_rates(engine, args.batch, args.context, T)

    shapes = {}
    if not (args.no_points or args.no_shapes) and args.preset == "llama3.2-1b" and layers == full_layers:
        import torch
        roof = decode_roofline(engine, args.batch, args.context, args.steps, sec)
        del engine      # its storage goes back before the wider shapes are built
        torch.cuda.empty_cache()
        for name in ("llama3.2-3b", "llama3.1-8b"):
            shapes.update(other_shape(name, args.dtype, args.batch, args.context, args.steps, args.warmup, T))   # timed as the headline is
        shapes.update(reference_bench_shapes(args.dtype))
    else:
        roof = decode_roofline(engine, args.batch, args.context, args.steps, sec)

    out = {
        "metric": "decode_tokens_per_second", "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": short,
        "data": "synthetic (seeded random weights N(0, 0.02), random token ids)",
        "config": {"model": args.preset, "batch": args.batch, "context": args.context, "layers": layers,
                   "layers_of_shape": full_layers, "hidden_size": cfg.hidden_size,
                   "intermediate_size": cfg.intermediate_size, "heads": cfg.num_attention_heads,
                   "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim, "vocab_size": cfg.vocab_size,
                   "tied_head": cfg.tie_word_embeddings, "page_size": page_size,
                   "sampling": "greedy" if args.temperature == 0 else f"temperature {args.temperature:g} top-p {args.top_p:g}",
                   "parallelism": "single GPU"},
        "step_ms_median": round(median * 1e3, 4),
        "prefill": {"value": round(T / psec, 1), "tokens": T, "ms": round(psec * 1e3, 3),
                    "frac": round(pflops / psec / MFMA_PEAK[short], 4)},
        "roofline": roof,
        "points": points, "workload_512_256": workload, "shapes": shapes, "measured": measured, "kernels": kernels,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
