"""The Llama-3 dense decoder as a plan of parts.

Embedding, N pre-norm blocks of grouped-query attention and SwiGLU, final RMS norm, output
projection (crates/burn-lm-llama/src/nn/transformer.rs:43-103, 189-256).  Two checkpoint
layouts are read, told apart by the name of the embedding tensor:

* Hugging Face names (``model.embed_tokens.weight`` ...; the name map of
  crates/burn-lm-llama/src/nn/llama/import.rs:35-88 read backwards).  Their q/k rows pair
  rotary lanes ``(i, i + head_dim/2)``; the reference permutes them on import
  (import.rs:94-127), here the rotary kernel pairs the lanes that way instead.
* Meta names (``tok_embeddings.weight`` ..., import.rs:20-33), already in the adjacent-pair
  layout of the reference's rotary table.
"""
from __future__ import annotations

import math

from ..config.llama import LlamaConfig
from ..parts.base import PartSpec
from ..registry import Architecture, register_architecture
from .plan import LayerPlan, ModelPlan, Place

HF_NAMES = dict(embedding="model.embed_tokens.weight", final_norm="model.norm.weight", head="lm_head.weight",
                layer="model.layers.{i}.", q="self_attn.q_proj.weight", k="self_attn.k_proj.weight",
                v="self_attn.v_proj.weight", o="self_attn.o_proj.weight", gate="mlp.gate_proj.weight",
                up="mlp.up_proj.weight", down="mlp.down_proj.weight", mixer_norm="input_layernorm.weight",
                ffn_norm="post_attention_layernorm.weight", pairing="half")
META_NAMES = dict(embedding="tok_embeddings.weight", final_norm="norm.weight", head="output.weight",
                  layer="layers.{i}.", q="attention.wq.weight", k="attention.wk.weight",
                  v="attention.wv.weight", o="attention.wo.weight", gate="feed_forward.w1.weight",
                  up="feed_forward.w3.weight", down="feed_forward.w2.weight", mixer_norm="attention_norm.weight",
                  ffn_norm="ffn_norm.weight", pairing="interleaved")


def plan(cfg: LlamaConfig, checkpoint_names=None) -> ModelPlan:
    n = META_NAMES if checkpoint_names is not None and META_NAMES["embedding"] in checkpoint_names else HF_NAMES
    d, hd = cfg.hidden_size, cfg.head_dim
    s = cfg.rope_scaling
    rope = PartSpec("rope", dict(
        head_dim=hd, theta=cfg.rope_theta, pairing=n["pairing"],
        scaling=None if s is None else (s.factor, s.low_freq_factor, s.high_freq_factor,
                                        s.original_max_position_embeddings)))
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = n["layer"].format(i=i)
        layers.append(LayerPlan(
            block="pre_norm",
            mixer=PartSpec("attention",
                           dict(width=d, heads=cfg.num_attention_heads, kv_heads=cfg.num_key_value_heads,
                                head_dim=hd, scale=1.0 / math.sqrt(hd), window=0),
                           dict(q=p + n["q"], k=p + n["k"], v=p + n["v"], o=p + n["o"])),
            feed_forward=PartSpec("swiglu", dict(width=d, inner=cfg.intermediate_size),
                                  dict(gate=p + n["gate"], up=p + n["up"], down=p + n["down"])),
            mixer_norm=PartSpec("rmsnorm", dict(width=d, eps=cfg.rms_norm_eps), dict(weight=p + n["mixer_norm"])),
            ffn_norm=PartSpec("rmsnorm", dict(width=d, eps=cfg.rms_norm_eps), dict(weight=p + n["ffn_norm"])),
            position="rope"))
    head_name = n["embedding"] if cfg.tie_word_embeddings else n["head"]
    return ModelPlan(
        vocab_size=cfg.vocab_size, width=d, max_positions=cfg.max_position_embeddings,
        embedding=PartSpec("table", dict(vocab=cfg.vocab_size, width=d), dict(weight=n["embedding"])),
        layers=layers, order=[Place(i) for i in range(cfg.num_hidden_layers)],
        final_norm=PartSpec("rmsnorm", dict(width=d, eps=cfg.rms_norm_eps), dict(weight=n["final_norm"])),
        head=PartSpec("linear", dict(vocab=cfg.vocab_size, width=d), dict(weight=head_name)),
        positions={"rope": rope}, stop_ids=tuple(cfg.eos_token_ids),
        ignorable_tensors=(r".*rotary_emb\.inv_freq$", r"^rope\.freqs$")
        + ((r"^lm_head\.weight$", r"^output\.weight$") if cfg.tie_word_embeddings else ()))


def checkpoint_tensors(cfg: LlamaConfig, names: str = "hf"):
    """Name -> (shape, role) of a fresh checkpoint of this configuration under Hugging Face names
    (``names="hf"``) or Meta names (``"meta"``: q/k rows in the adjacent-pair order)."""
    if names not in ("hf", "meta"):
        raise ValueError(f"checkpoint names {names!r} unknown; 'hf' or 'meta'")
    n = HF_NAMES if names == "hf" else META_NAMES
    d, hd = cfg.hidden_size, cfg.head_dim
    out = {n["embedding"]: ((cfg.vocab_size, d), "table")}
    for i in range(cfg.num_hidden_layers):
        p = n["layer"].format(i=i)
        out[p + n["mixer_norm"]] = ((d,), "norm")
        out[p + n["q"]] = ((cfg.num_attention_heads * hd, d), "matrix")
        out[p + n["k"]] = ((cfg.num_key_value_heads * hd, d), "matrix")
        out[p + n["v"]] = ((cfg.num_key_value_heads * hd, d), "matrix")
        out[p + n["o"]] = ((d, cfg.num_attention_heads * hd), "matrix")
        out[p + n["ffn_norm"]] = ((d,), "norm")
        out[p + n["gate"]] = ((cfg.intermediate_size, d), "matrix")
        out[p + n["up"]] = ((cfg.intermediate_size, d), "matrix")
        out[p + n["down"]] = ((d, cfg.intermediate_size), "matrix")
    out[n["final_norm"]] = ((d,), "norm")
    if not cfg.tie_word_embeddings:
        out[n["head"]] = ((cfg.vocab_size, d), "matrix")
    return out


def chat_template(messages) -> str:
    """The Llama-3 chat framing of crates/burn-lm-llama/src/server/llama3.rs:561-576: every message
    under a header with its role, closed by ``<|eot_id|>``, then the header of the assistant's turn."""
    out = "".join(f"<|start_header_id|>{m['role'].lower()}<|end_header_id|>\n\n{m['content']}<|eot_id|>"
                  for m in messages)
    return out + "<|start_header_id|>assistant<|end_header_id|>\n\n"


# the special tokens the reference's Llama-3 tokenizer knows by name and stops at
# (crates/burn-lm-llama/src/tokenizer/tiktoken.rs:12-15, 126-132)
SPECIAL_TOKENS = dict(bos="<|begin_of_text|>", eos="<|end_of_text|>",
                      stops=("<|end_of_text|>", "<|eom_id|>", "<|eot_id|>"))

LLAMA = Architecture(name="LlamaForCausalLM", read_config=LlamaConfig.from_dict, plan=plan,
                     checkpoint_tensors=checkpoint_tensors, display_name="Llama 3", created_by="Meta",
                     chat_template=chat_template, special_tokens=SPECIAL_TOKENS)
register_architecture(LLAMA, "llama")
