"""Decode and prefill throughput of the engine on one MI355X, with roofline fractions.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 4096] [--layers L]
    python bench.py --preset llama3.2-3b --unequal 16 [--generate 256]     (an unequal batch, end to end)

A "step" is one decode step of the whole batch: the engine's step function on one token per
sequence, the sampling kernel, and the tokens' trip to the host, as the generation loop does it.
The default run has the layer sizes of the Llama-3.2-1B shape with random weights, a batch of 8
and a context of 4096 tokens per sequence.  One JSON line is printed.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0                                   # MI355X HBM3E, published
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}          # dense, published


def weight_bytes(cfg, layers, itemsize):
    d, hd = cfg.hidden_size, cfg.head_dim
    per_layer = ((cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * hd * d + d * cfg.num_attention_heads * hd
                 + 3 * cfg.intermediate_size * d + 2 * d)
    head = cfg.vocab_size * d
    return (layers * per_layer + d + head) * itemsize   # the embedding rows read are negligible; tied or not, the head is read once


def kv_bytes_per_token(cfg, layers, itemsize):
    return 2 * layers * cfg.num_key_value_heads * cfg.head_dim * itemsize


def prefill_flops(cfg, layers, T, rows_out=1):
    d, hd, nh, nkv = cfg.hidden_size, cfg.head_dim, cfg.num_attention_heads, cfg.num_key_value_heads
    lin = 2 * T * ((nh + 2 * nkv) * hd * d + d * nh * hd + 3 * cfg.intermediate_size * d)
    attn = 2 * 2 * nh * hd * (T * (T + 1) // 2)
    return layers * (lin + attn) + 2 * rows_out * cfg.vocab_size * d


def fill_cache(engine, n_seqs, length, seed=0):
    """Sequences that already hold `length` tokens: pages reserved, lengths set, keys and values
    random (synthetic; what they hold does not change the work of a decode step)."""
    import torch
    g = torch.Generator(device=engine.rt.device).manual_seed(seed)
    for grp in engine.cache.groups:
        grp.storage.normal_(0.0, 1.0, generator=g)
    slots = []
    for _ in range(n_seqs):
        s = engine.open()
        engine.cache.reserve([(s, length)])
        engine.cache.advance(s, length)
        slots.append(s)
    return slots


def time_decode(engine, sampler, batch, context, steps, warmup):
    import torch
    for s in list(engine.cache.live_slots):
        engine.close(s)
    start = context - (steps + warmup + 1)
    slots = fill_cache(engine, batch, start)
    reqs = list(range(batch))
    rows = list(range(batch))

    def run(n, first_index, picked):
        """n decode steps the way the generation loop runs them: the next step starts from the tokens
        left on the GPU, then the host reads the tokens of the step before."""
        for i in range(n):
            logits = engine.step_ahead(slots, rows, picked)
            if logits is None:      # a shape without a recorded graph yet: the plain step, which records it
                logits = engine.step([(s, [t], [0]) for s, t in zip(slots, picked.tokens())])
            nxt = sampler.pick_device(logits, reqs, [first_index + i] * batch)
            picked.tokens()
            picked = nxt
        return picked

    logits = engine.step([(s, [1], [0]) for s in slots])
    picked = run(warmup, 0, sampler.pick_device(logits, reqs, [0] * batch))
    picked.tokens()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    picked = run(steps, warmup, picked)
    picked.tokens()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    for s in slots:
        engine.close(s)
    return dt / steps


def time_prefill(engine, T, reps=3):
    import torch
    import numpy as np
    toks = [int(x) for x in np.random.default_rng(0).integers(0, engine.vocab_size, T)]
    best = None
    for r in range(reps + 1):
        s = engine.open()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([(s, toks, [T - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        engine.close(s)
        if r > 0:
            best = dt if best is None else min(best, dt)
    return best


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
    for _ in range(3):      # the first run records the graphs of its shapes
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
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and batch 64 decode points")
    ap.add_argument("--temperature", type=float, default=0.0, help="sample instead of picking greedily (0: greedy)")
    ap.add_argument("--top-p", type=float, default=1.0, help="nucleus mass when sampling")
    ap.add_argument("--unequal", type=int, default=0, metavar="N",
                    help="instead of the decode measurement: N prompts of 64..2048 tokens through the generation loop")
    ap.add_argument("--generate", type=int, default=256, help="tokens generated per prompt with --unequal")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this library has no multi-GPU path (run with --gpus 1)")
        sys.exit(2)

    if args.unequal:
        return run_unequal(args)

    import torch
    from burn_lm_amd.config.presets import preset
    from burn_lm_amd.engine.loading import random_engine
    from burn_lm_amd.sampling.sampler import Sampler

    config = preset(args.preset)
    full_layers = config["num_hidden_layers"]
    layers = args.layers or full_layers
    config["num_hidden_layers"] = layers
    biggest = max(args.batch, 1 if args.no_points else 64)
    engine = random_engine(config, seed=0, dtype=args.dtype, max_tokens=biggest * args.context,
                           max_seqs=biggest, max_context=args.context)
    cfg = engine.config
    itemsize = 2 if args.dtype == "bfloat16" else 4
    sampler = Sampler(temperature=args.temperature, top_p=args.top_p, seed=1)

    sec = time_decode(engine, sampler, args.batch, args.context, args.steps, args.warmup)
    value = args.batch / sec
    mean_ctx = args.context - args.steps / 2
    step_bytes = weight_bytes(cfg, layers, itemsize) + kv_bytes_per_token(cfg, layers, itemsize) * mean_ctx * args.batch
    achieved = step_bytes / sec / 1e9

    T = args.prefill_tokens
    psec = time_prefill(engine, T)
    pf = prefill_flops(cfg, layers, T)
    peak = MFMA_PEAK["bf16" if args.dtype == "bfloat16" else "fp32"]

    points = {}
    if not args.no_points:
        for b in (1, 64):
            s = time_decode(engine, sampler, b, args.context, max(8, args.steps // 2), 4)
            points[f"decode_b{b}"] = round(b / s, 1)

    out = {
        "metric": "decode_tokens_per_second", "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic (seeded random weights N(0, 0.02), random token ids, random cache contents)",
        "config": {"model": args.preset, "batch": args.batch, "context": args.context, "layers": layers,
                   "layers_of_shape": full_layers, "hidden_size": cfg.hidden_size,
                   "intermediate_size": cfg.intermediate_size, "heads": cfg.num_attention_heads,
                   "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim, "vocab_size": cfg.vocab_size,
                   "tied_head": cfg.tie_word_embeddings, "page_size": engine.cache.page_size,
                   "sampling": "greedy" if args.temperature == 0 else f"temperature {args.temperature:g} top-p {args.top_p:g}",
                   "parallelism": "single GPU"},
        "prefill": {"value": round(T / psec, 1), "tokens": T, "ms": round(psec * 1e3, 3), "frac": round(pf / psec / peak, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": points,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
