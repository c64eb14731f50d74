"""Plain, slow Llama-3 decoder in numpy float64: whole sequences, no cache, one function per part.

Written from the formulas of tracel-ai/burn-lm (paths relative to the reference root,
``LL/`` = ``crates/burn-lm-llama/src/``).  It shares no code with the product package:
it has its own folder reader, its own weight re-layout and its own maths.  The reference
keeps linear weights as ``[d_in, d_out]`` (``y = x @ W``); checkpoints keep
``[d_out, d_in]``, so every projection here is ``x @ W.T`` on the checkpoint matrix.

Rotary pairing follows the reference: *adjacent* lanes ``(x[2i], x[2i+1])`` form a pair
(``freq_complex`` table, LL/nn/pos_encoding.rs:25) and checkpoints in the Hugging Face
layout have the rows of their q/k projections permuted into that order first
(LL/nn/llama/import.rs:94-127).
"""
from __future__ import annotations

import json
import math
import os

import numpy as np


# ----------------------------------------------------------------------------------------
# optional rounding: where a bfloat16 engine rounds, so that its tests can be tight
# ----------------------------------------------------------------------------------------
def round_bf16(x):
    """Nearest-even rounding of float64 values to bfloat16 (8 significant bits), returned as float64."""
    a = np.ascontiguousarray(np.asarray(x, dtype=np.float64).astype(np.float32))
    u = a.view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).astype(np.float64).reshape(a.shape)


class Rounding:
    """Where values are rounded to bfloat16 between the exact formulas.  Always: the normalised
    activations, q and k after the rotation, v, the attention output, the gated product, the final
    norm's output.  The residual stream and its sums, the statistics of norms and softmax, and all
    products' sums stay exact.  Options say whether a value is rounded as well, each one flag or
    one flag per token of the sequence (a token keeps the flags of the step that fed it):
    ``projections`` (q and k before their rotation), ``gate_up`` (gate and up before the gating),
    ``attention_delta`` and ``feed_forward_delta`` (the output and the down projection before they
    are added to the residual stream): an engine rounds there where it runs the steps as separate
    kernels and not where it fuses them or hands on unrounded partial sums;
    ``probabilities``: the softmax weights ``exp(score - maximum)`` before they multiply the values
    and are summed, relative to the row's maximum; or, when keys are visited in pages of
    ``probability_pages``, relative to the maximum of the pages up to the key's own
    (``running_maximum``, one page after the other) or of the key's own page alone (every page on
    its own), the weights then being scaled, exactly, to the row's maximum."""

    def __init__(self, projections=True, gate_up=True, attention_delta=True, feed_forward_delta=True,
                 probabilities=True, probability_pages=None, running_maximum=True):
        self.projections, self.gate_up = projections, gate_up
        self.attention_delta, self.feed_forward_delta = attention_delta, feed_forward_delta
        self.probabilities, self.probability_pages, self.running_maximum = probabilities, probability_pages, running_maximum

    r = staticmethod(round_bf16)


def _r(rounding, x, when=True, token_axis=None):
    """x rounded if a rounding is given and ``when`` holds; ``when`` may hold one flag per token,
    x's axis ``token_axis`` then runs over the tokens."""
    if rounding is None or when is False:
        return x
    if when is True:
        return rounding.r(x)
    flags = np.asarray(when, dtype=bool)
    shape = [1] * np.ndim(x)
    shape[token_axis] = flags.shape[0]
    return np.where(flags.reshape(shape), rounding.r(x), x)


# ----------------------------------------------------------------------------------------
# parts
# ----------------------------------------------------------------------------------------
def rms_norm(x, gamma, eps):
    """y = x / sqrt(mean(x^2) + eps) * gamma over the last axis.

    LL/nn/transformer.rs:60-62 (epsilon passed to every norm), vector at :278-297.
    """
    x = np.asarray(x, dtype=np.float64)
    ms = np.mean(x * x, axis=-1, keepdims=True)
    return x / np.sqrt(ms + eps) * np.asarray(gamma, dtype=np.float64)


def rope_base_frequencies(head_dim, theta):
    """theta_i = theta^(-2i/head_dim), i = 0..head_dim/2-1 (LL/nn/llama/base.rs:273-284)."""
    i = np.arange(0, head_dim, 2, dtype=np.float64)
    return 1.0 / (float(theta) ** (i / head_dim))


def llama3_frequency_scaling(freqs, scale_factor=8.0, low_freq_factor=1.0,
                             high_freq_factor=4.0, old_context_len=8192.0):
    """Llama-3.1 "by parts" scaling, mask by mask as LL/nn/pos_encoding.rs:107-138.

    Defaults are those of ``RopeFrequencyScaling`` (LL/nn/pos_encoding.rs:91-101).
    """
    freqs = np.asarray(freqs, dtype=np.float64)
    low_freq_wavelen = old_context_len / low_freq_factor
    high_freq_wavelen = old_context_len / high_freq_factor
    wavelen = 2.0 * math.pi / freqs
    smooth = (old_context_len / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
    blended = (1.0 - smooth) * freqs / scale_factor + smooth * freqs
    new = np.where(wavelen >= high_freq_wavelen, blended, freqs)      # :113-128
    new = np.where(wavelen > low_freq_wavelen, freqs / scale_factor, new)  # :130-132
    new = np.where(wavelen < high_freq_wavelen, freqs, new)          # :134-137
    return new


def rope_interleaved(x, positions, freqs):
    """Rotate adjacent pairs of the last axis by ``position * freq`` radians.

    x: [..., T, head_dim]; positions: [T] absolute positions (LL/nn/pos_encoding.rs:66-79);
    vector at LL/nn/pos_encoding.rs:165-174 (position 0 identity, position 1 turns the
    pair (x0, x1) by 1 rad when theta_0 = 1).
    """
    x = np.asarray(x, dtype=np.float64)
    ang = np.asarray(positions, dtype=np.float64)[:, None] * np.asarray(freqs)[None, :]
    c, s = np.cos(ang), np.sin(ang)
    x0, x1 = x[..., 0::2], x[..., 1::2]
    out = np.empty_like(x)
    out[..., 0::2] = x0 * c - x1 * s
    out[..., 1::2] = x0 * s + x1 * c
    return out


def permute_hf_rows(w, n_heads):
    """Hugging Face q/k projection rows -> the interleaved pair order.

    The reference does ``reshape [d_in, heads, 2, hd/2] -> swap(2,3) -> reshape`` on the
    ``[d_in, d_out]`` matrix (LL/nn/llama/import.rs:99-126); on a ``[d_out, d_in]``
    checkpoint matrix the same move acts on the rows.
    """
    d_out, d_in = w.shape
    hd = d_out // n_heads
    return w.reshape(n_heads, 2, hd // 2, d_in).swapaxes(1, 2).reshape(d_out, d_in)


def repeat_kv(x, n_rep):
    """[B, nkv, S, hd] -> [B, nkv*n_rep, S, hd]; query head h uses KV head h // n_rep
    (LL/nn/attention/mha.rs:174-185)."""
    if n_rep == 1:
        return x
    b, nkv, s, hd = x.shape
    return np.broadcast_to(x[:, :, None], (b, nkv, n_rep, s, hd)).reshape(b, nkv * n_rep, s, hd)


def hidden_mask(t, s):
    """True = hidden: key j is hidden from query i when j > i + (s - t)
    (LL/nn/transformer.rs:168-180; none at all when t <= 1)."""
    if t <= 1:
        return None
    i = np.arange(t)[:, None]
    j = np.arange(s)[None, :]
    return j > i + (s - t)


def softmax(x, axis=-1):
    x = x - np.max(x, axis=axis, keepdims=True)
    e = np.exp(x)
    return e / np.sum(e, axis=axis, keepdims=True)


def scaled_attention(q, k, v, mask, rounding=None):
    """softmax(q k^T / sqrt(hd) + mask) v with the scale applied to the product
    (LL/nn/attention/mha.rs:143-171).  q [B,nh,T,hd]; k, v [B,nkv,S,hd]."""
    n_rep = q.shape[1] // k.shape[1]
    k = repeat_kv(k, n_rep)
    v = repeat_kv(v, n_rep)
    scores = np.matmul(q, np.swapaxes(k, 2, 3)) / math.sqrt(q.shape[-1])
    if mask is not None:
        scores = np.where(mask[None, None], -np.inf, scores)
    if rounding is None or rounding.probabilities is False:
        return np.matmul(softmax(scores, axis=3), v)
    final = np.max(scores, axis=3, keepdims=True)
    seen = final
    if rounding.probability_pages:      # the maximum of the pages up to and including each key's own
        n = rounding.probability_pages
        pages = [np.max(scores[..., a:a + n], axis=3, keepdims=True) for a in range(0, scores.shape[3], n)]
        own = np.concatenate(pages, axis=3)
        running = np.maximum.accumulate(own, axis=3)
        if rounding.running_maximum is not True:
            flags = np.broadcast_to(np.asarray(rounding.running_maximum, dtype=bool), (scores.shape[2],))
            running = np.where(flags.reshape(1, 1, -1, 1), running, own)
        seen = np.repeat(running, n, axis=3)[..., :scores.shape[3]]
        seen = np.where(np.isfinite(seen), seen, final)     # pages of which a query sees nothing
    e = np.exp(scores - seen)                                   # weights in (0, 1]
    e = _r(rounding, e, rounding.probabilities, token_axis=2) * np.exp(seen - final)
    return np.matmul(e, v) / np.sum(e, axis=3, keepdims=True)


def attention_layer(x, wq, wk, wv, wo, n_heads, n_kv_heads, head_dim, freqs, start_pos=0, rounding=None):
    """Whole-sequence attention sub-layer without cache (``forward_masked``,
    LL/nn/attention/mha.rs:50-69; projections :121-140).  x [B,T,D]; weights
    ``[d_out, d_in]`` already in the interleaved pair order."""
    b, t, _ = x.shape
    q = (x @ wq.T).reshape(b, t, n_heads, head_dim).swapaxes(1, 2)
    k = (x @ wk.T).reshape(b, t, n_kv_heads, head_dim).swapaxes(1, 2)
    v = (x @ wv.T).reshape(b, t, n_kv_heads, head_dim).swapaxes(1, 2)
    if rounding is not None:
        q, k = _r(rounding, q, rounding.projections, 2), _r(rounding, k, rounding.projections, 2)
        v = rounding.r(v)
    pos = np.arange(start_pos, start_pos + t)
    q = _r(rounding, rope_interleaved(q, pos, freqs))
    k = _r(rounding, rope_interleaved(k, pos, freqs))
    o = _r(rounding, scaled_attention(q, k, v, hidden_mask(t, t), rounding))
    o = o.swapaxes(1, 2).reshape(b, t, n_heads * head_dim)
    return o @ wo.T if rounding is None else _r(rounding, o @ wo.T, rounding.attention_delta, 1)


def silu(z):
    return z / (1.0 + np.exp(-z))


def swiglu_feed_forward(x, w_gate, w_up, w_down, rounding=None):
    """(silu(x W1) * (x W3)) W2 (LL/nn/fftn.rs:44-46; W1 = swiglu.linear_inner = gate,
    W3 = swiglu.linear_outer = up, LL/nn/llama/import.rs:22-31).  Vector at fftn.rs:57-92."""
    if rounding is None:
        return (silu(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T
    g, u = _r(rounding, x @ w_gate.T, rounding.gate_up, 1), _r(rounding, x @ w_up.T, rounding.gate_up, 1)
    return _r(rounding, rounding.r(silu(g) * u) @ w_down.T, rounding.feed_forward_delta, 1)


def block(x, lw, cfg, freqs, start_pos=0, rounding=None):
    """h = x + attn(norm1(x)); out = h + ffn(norm2(h)) (LL/nn/transformer.rs:241-256)."""
    h = x + attention_layer(_r(rounding, rms_norm(x, lw["attention_norm"], cfg["eps"])),
                            lw["wq"], lw["wk"], lw["wv"], lw["wo"],
                            cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"], freqs, start_pos, rounding)
    return h + swiglu_feed_forward(_r(rounding, rms_norm(h, lw["ffn_norm"], cfg["eps"])),
                                   lw["w1"], lw["w3"], lw["w2"], rounding)


def transformer_forward(ids, model, start_pos=0, rounding=None):
    """Embedding -> blocks -> final norm -> output projection, logits for every position
    (LL/nn/transformer.rs:88-103).  ids [B,T] ints; returns [B,T,V] float64.  With a ``Rounding``
    the values a bfloat16 engine keeps in bfloat16 are rounded on the way (the formulas stay these)."""
    cfg = model["cfg"]
    ids = np.asarray(ids)
    h = model["tok_embeddings"][ids]
    for lw in model["layers"]:
        h = block(h, lw, cfg, model["freqs"], start_pos, rounding)
    h = _r(rounding, rms_norm(h, model["norm"], cfg["eps"]))
    return h @ model["output"].T


# ----------------------------------------------------------------------------------------
# sampling
# ----------------------------------------------------------------------------------------
def temperature_softmax(logits, temperature):
    """softmax(logits / temperature) (LL/generation/generate.rs:8-10; vector :121-137)."""
    return softmax(np.asarray(logits, dtype=np.float64) / temperature, axis=-1)


def top_p_keep(probs, p):
    """Indices kept by the reference's nucleus rule: sort descending, keep a token while
    the mass *before* it is < p (LL/generation/sampling.rs:50-63)."""
    order = np.argsort(-np.asarray(probs), kind="stable")
    kept, cum = [], 0.0
    for i in order:
        if cum >= p:
            break
        kept.append(int(i))
        cum += float(probs[i])
    return kept


def greedy_generate(model, prompt, n_new, stop_ids=()):
    """Argmax continuation by re-running the whole sequence each time
    (loop of LL/generation/generate.rs:61-98 with Sampler::Argmax, sampling.rs:18).
    The stop token is produced and then ends the sequence (generation/context.rs:142-170)."""
    toks = list(prompt)
    out = []
    for _ in range(n_new):
        logits = transformer_forward([toks], model)[0, -1]
        nxt = int(np.argmax(logits))
        out.append(nxt)
        toks.append(nxt)
        if nxt in stop_ids:
            break
    return out


# ----------------------------------------------------------------------------------------
# model folder -> plain model (own reader; Hugging Face tensor names)
# ----------------------------------------------------------------------------------------
def _read_safetensors(path):
    """Minimal reader: 8-byte little-endian header length, JSON header, raw data."""
    with open(path, "rb") as f:
        n = int.from_bytes(f.read(8), "little")
        header = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        a, b = meta["data_offsets"]
        raw = data[a:b]
        dt = meta["dtype"]
        if dt == "F32":
            arr = np.frombuffer(raw, dtype="<f4").astype(np.float64)
        elif dt == "BF16":
            u = np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16
            arr = u.view(np.float32).astype(np.float64)
        elif dt == "F16":
            arr = np.frombuffer(raw, dtype="<f2").astype(np.float64)
        else:
            raise ValueError(f"plain reader: dtype {dt} of {name}")
        out[name] = arr.reshape(meta["shape"])
    return out


def load_model_folder(folder):
    """Read config.json + model.safetensors (Hugging Face names) into the plain model.

    Name map and q/k row permutation as LL/nn/llama/import.rs:35-88 and :94-127; field
    defaults as LL/nn/llama/base.rs:40-71 (kv heads default to heads :254, head_dim =
    d_model / heads, LL/nn/attention/mha.rs:191).
    """
    with open(os.path.join(folder, "config.json")) as f:
        c = json.load(f)
    t = _read_safetensors(os.path.join(folder, "model.safetensors"))
    nh = c["num_attention_heads"]
    nkv = c.get("num_key_value_heads", nh)
    hd = c.get("head_dim") or c["hidden_size"] // nh
    cfg = dict(n_heads=nh, n_kv_heads=nkv, head_dim=hd, eps=c.get("rms_norm_eps", 1e-5))
    freqs = rope_base_frequencies(hd, c.get("rope_theta", 10000.0))
    rs = c.get("rope_scaling")
    if rs:
        freqs = llama3_frequency_scaling(
            freqs, rs.get("factor", 8.0), rs.get("low_freq_factor", 1.0),
            rs.get("high_freq_factor", 4.0), rs.get("original_max_position_embeddings", 8192))
    layers = []
    for i in range(c["num_hidden_layers"]):
        p = f"model.layers.{i}."
        layers.append(dict(
            wq=permute_hf_rows(t[p + "self_attn.q_proj.weight"], nh),
            wk=permute_hf_rows(t[p + "self_attn.k_proj.weight"], nkv),
            wv=t[p + "self_attn.v_proj.weight"],
            wo=t[p + "self_attn.o_proj.weight"],
            w1=t[p + "mlp.gate_proj.weight"],
            w3=t[p + "mlp.up_proj.weight"],
            w2=t[p + "mlp.down_proj.weight"],
            attention_norm=t[p + "input_layernorm.weight"],
            ffn_norm=t[p + "post_attention_layernorm.weight"],
        ))
    emb = t["model.embed_tokens.weight"]
    out = emb if c.get("tie_word_embeddings", False) else t["lm_head.weight"]
    return dict(cfg=cfg, freqs=freqs, tok_embeddings=emb, layers=layers,
                norm=t["model.norm.weight"], output=out, vocab=c["vocab_size"])
