"""Shared by the tests: two tiny configurations that differ in every size and option and a middle-sized one, model
folders with random weights in a temporary place, and a builder of replay traces."""
import json
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# A: grouped heads (2 per group), head size 16, tied head, no frequency scaling
TINY_A = dict(architectures=["LlamaForCausalLM"], model_type="llama", hidden_size=64, intermediate_size=176,
              num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, vocab_size=256,
              max_position_embeddings=1024, rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=True)
# B: one key-value head for six query heads, head size 24 (no power of two, not width/heads * anything
# special), widths and vocabulary that are no powers of two, another eps, llama3 scaling whose three
# branches are all hit at head size 24, separate head
TINY_B = dict(architectures=["LlamaForCausalLM"], model_type="llama", hidden_size=144, intermediate_size=384,
              num_hidden_layers=3, num_attention_heads=6, num_key_value_heads=1, head_dim=24, vocab_size=384,
              max_position_embeddings=384, rms_norm_eps=1e-6, rope_theta=500000.0, tie_word_embeddings=False,
              rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                original_max_position_embeddings=32))
# C: middle-sized, so that the matrix-core paths run (skinny products on packed weights, the fused
# q/k/v projection, attention with head size 64 and four query heads per group, cut sequences): the
# Llama-3.2 frequency scaling as published (factor 32, original context 8192), tied head
MID_C = dict(architectures=["LlamaForCausalLM"], model_type="llama", hidden_size=512, intermediate_size=1408,
             num_hidden_layers=2, num_attention_heads=8, num_key_value_heads=2, vocab_size=5000,
             max_position_embeddings=4096, rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=True,
             rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                               original_max_position_embeddings=8192))
TINIES = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (MID_C, 2)}

# logits are compared as max |difference| relative to max |expected|
TOL = {"float32": 1e-5, "bfloat16": 3e-2}


def make_folder(path, cfg, seed, std=None, norm_jitter=0.1, **kw):
    """Weights N(0, std).  The tiny models take 0.08, so that their logits are far from uniform; at
    width 512 that scale sharpens the attention so much that bfloat16 activations alone (exact
    arithmetic between the roundings, on the CPU) put 1 logit row in 100 at 0.024 of the largest
    logit and the worst of 2,400 at 0.029, the tolerance's edge; at 0.05 those are 0.014 and 0.017."""
    import burn_lm_amd
    if std is None:
        std = 0.05 if cfg is MID_C else 0.08
    return burn_lm_amd.write_random_model(str(path), cfg, seed=seed, std=std, norm_jitter=norm_jitter, **kw)


def random_tokens(seed, vocab, n):
    return [int(x) for x in np.random.default_rng(seed).integers(0, vocab, n)]


def rel_err(got, want):
    return float(np.abs(np.asarray(got, dtype=np.float64) - want).max() / max(1e-30, np.abs(want).max()))


class Trace:
    """Collects steps for bin/trace_run and remembers which (request, position) each wanted row is, and
    for each step and request how the request's tokens so far were fed (history)."""

    def __init__(self):
        self.lines, self.index, self.n = [], {}, 0
        self.live, self.peak = {}, 0
        self.fed_by, self.history = {}, {}

    def step(self, entries, end=()):
        """entries: (request id, start position, tokens, want list)."""
        rows = []
        total = sum(len(toks) for _, _, toks, _ in entries)
        for rid, start, toks, want in entries:
            rows += [(rid, start + w) for w in want]
            self.live[rid] = start + len(toks)
            # for every token the request holds, the rows of the step that fed it and whether it came alone
            self.fed_by[rid] = (self.fed_by[rid] if start else []) + [(total, len(toks) == 1 and start > 0)] * len(toks)
            if want:
                self.history[self.n, rid] = list(self.fed_by[rid])
        self.peak = max(self.peak, sum((n + 63) // 64 * 64 for n in self.live.values()))
        for rid in end:
            self.live.pop(rid)
        self.lines.append(json.dumps({"step": self.n, "entries": [
            {"id": rid, "tokens": toks, "want": want} for rid, _, toks, want in entries], "end": list(end)}))
        if rows:
            self.index[self.n] = rows
        self.n += 1

    def text(self):
        return "\n".join(self.lines) + "\n"


def run_trace(folder, dtype, trace, out_dir, max_tokens=None, timeout=600):
    """Runs bin/trace_run as a user would and returns {step: float32 array [wanted, vocab]}."""
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(folder), "--dtype", dtype,
           "--out", str(out_dir), "--max-tokens", str(max_tokens or trace.peak)]
    r = subprocess.run(cmd, input=trace.text(), capture_output=True, text=True, timeout=timeout)
    assert r.returncode == 0, f"trace_run failed ({r.returncode}):\n{r.stdout[-2000:]}\n{r.stderr[-4000:]}"
    done = [l for l in r.stdout.splitlines() if l.startswith("done ")]
    assert [int(l.split()[1]) for l in done] == list(range(trace.n)), "a 'done <step>' line is missing"
    with open(os.path.join(folder, "config.json")) as f:
        vocab = json.load(f)["vocab_size"]
    out = {}
    for s, rows in trace.index.items():
        a = np.fromfile(os.path.join(out_dir, f"{s}.f32"), dtype="<f4")
        assert a.size == len(rows) * vocab, f"step {s}: {a.size} floats for {len(rows)} rows of {vocab}"
        out[s] = a.reshape(len(rows), vocab)
    return out
