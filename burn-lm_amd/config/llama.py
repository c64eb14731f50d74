"""Typed configuration of the Llama-3 decoder, read from the keys of its ``config.json``.

The reference keeps its model shapes as presets in code (crates/burn-lm-llama/src/nn/llama/
base.rs:40-139) and has no reader for ``config.json``; the fields here are the same ones under
their Hugging Face key names, and defaults for optional keys are the reference's own
(``norm_eps`` 1e-5 base.rs:57-59, RoPE theta 10000 base.rs:61-62, key-value heads = heads
base.rs:254, head size = width / heads nn/attention/mha.rs:191, frequency-scaling factors
nn/pos_encoding.rs:91-101).  Every size is a required key: none is assumed.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Optional, Tuple

from ..errors import ConfigError  # noqa: F401  (also imported from here by older callers)


@dataclass(frozen=True)
class RopeScaling:
    """llama3 "by parts" frequency scaling (crates/burn-lm-llama/src/nn/pos_encoding.rs:91-138)."""
    factor: float = 8.0
    low_freq_factor: float = 1.0
    high_freq_factor: float = 4.0
    original_max_position_embeddings: int = 8192


def _need(d, key, kind, where="config.json"):
    if key not in d or d[key] is None:
        raise ConfigError(f"{where}: required key '{key}' is missing")
    return _typed(d, key, kind, where)


def _typed(d, key, kind, where="config.json"):
    v = d[key]
    if kind is int:
        if isinstance(v, bool) or not isinstance(v, int):
            raise ConfigError(f"{where}: key '{key}' must be an integer, got {v!r}")
        return v
    if kind is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{where}: key '{key}' must be a number, got {v!r}")
        return float(v)
    if kind is bool:
        if not isinstance(v, bool):
            raise ConfigError(f"{where}: key '{key}' must be true or false, got {v!r}")
        return v
    raise AssertionError(kind)


def _token_ids(d, key):
    v = d.get(key)
    if v is None:
        return ()
    if isinstance(v, int) and not isinstance(v, bool):
        return (v,)
    if isinstance(v, list) and all(isinstance(x, int) and not isinstance(x, bool) for x in v):
        return tuple(v)
    raise ConfigError(f"config.json: key '{key}' must be an integer or a list of integers, got {v!r}")


@dataclass(frozen=True)
class LlamaConfig:
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    max_position_embeddings: int
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    rope_scaling: Optional[RopeScaling] = None
    tie_word_embeddings: bool = False
    bos_token_id: Optional[int] = None
    eos_token_ids: Tuple[int, ...] = ()
    torch_dtype: str = "bfloat16"
    architecture: str = "LlamaForCausalLM"
    extra: dict = field(default_factory=dict, compare=False, hash=False)

    # -------------------------------------------------------------------------------------
    @staticmethod
    def from_dict(d: dict) -> "LlamaConfig":
        if not isinstance(d, dict):
            raise ConfigError("config.json must hold a JSON object")
        hidden = _need(d, "hidden_size", int)
        heads = _need(d, "num_attention_heads", int)
        kv_heads = _typed(d, "num_key_value_heads", int) if d.get("num_key_value_heads") is not None else heads
        if heads <= 0 or hidden <= 0:
            raise ConfigError("config.json: 'hidden_size' and 'num_attention_heads' must be positive")
        if d.get("head_dim") is not None:
            head_dim = _typed(d, "head_dim", int)
        else:
            if hidden % heads:
                raise ConfigError(f"config.json: 'hidden_size' {hidden} is not a multiple of "
                                  f"'num_attention_heads' {heads} and no 'head_dim' is given")
            head_dim = hidden // heads
        scaling = None
        rs = d.get("rope_scaling")
        if rs is not None:
            if not isinstance(rs, dict):
                raise ConfigError("config.json: 'rope_scaling' must be null or an object")
            kind = rs.get("rope_type", rs.get("type"))
            if kind not in ("llama3", "default"):
                raise ConfigError(f"config.json: rope_scaling.rope_type {kind!r} is not supported "
                                  f"(only 'llama3', or 'default' for none)")
            dflt = RopeScaling()
            w = "config.json rope_scaling"
            scaling = RopeScaling(
                factor=_typed(rs, "factor", float, w) if "factor" in rs else dflt.factor,
                low_freq_factor=_typed(rs, "low_freq_factor", float, w) if "low_freq_factor" in rs else dflt.low_freq_factor,
                high_freq_factor=_typed(rs, "high_freq_factor", float, w) if "high_freq_factor" in rs else dflt.high_freq_factor,
                original_max_position_embeddings=(_typed(rs, "original_max_position_embeddings", int, w)
                                                  if "original_max_position_embeddings" in rs
                                                  else dflt.original_max_position_embeddings))
            if kind == "default":   # the plain frequencies, spelled out
                scaling = None
        # the architecture has no bias and one activation (crates/burn-lm-llama/src/nn/attention/
        # mha.rs:193-204, nn/fftn.rs:27-32): say so instead of silently ignoring the keys
        for key in ("attention_bias", "mlp_bias"):
            if d.get(key):
                raise ConfigError(f"config.json: '{key}' is true, but this architecture has no bias terms")
        if d.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"config.json: 'hidden_act' {d['hidden_act']!r} is not supported (only 'silu')")
        archs = d.get("architectures")
        arch = archs[0] if isinstance(archs, list) and archs else d.get("model_type", "LlamaForCausalLM")
        bos = d.get("bos_token_id")
        if bos is not None and (isinstance(bos, bool) or not isinstance(bos, int)):
            raise ConfigError(f"config.json: key 'bos_token_id' must be an integer, got {bos!r}")
        known = {"hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                 "num_key_value_heads", "head_dim", "vocab_size", "max_position_embeddings", "rms_norm_eps",
                 "rope_theta", "rope_scaling", "tie_word_embeddings", "bos_token_id", "eos_token_id",
                 "torch_dtype", "architectures", "model_type", "attention_bias", "mlp_bias", "hidden_act"}
        cfg = LlamaConfig(
            hidden_size=hidden,
            intermediate_size=_need(d, "intermediate_size", int),
            num_hidden_layers=_need(d, "num_hidden_layers", int),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            vocab_size=_need(d, "vocab_size", int),
            max_position_embeddings=_need(d, "max_position_embeddings", int),
            rms_norm_eps=_typed(d, "rms_norm_eps", float) if d.get("rms_norm_eps") is not None else 1e-5,
            rope_theta=_typed(d, "rope_theta", float) if d.get("rope_theta") is not None else 10000.0,
            rope_scaling=scaling,
            tie_word_embeddings=_typed(d, "tie_word_embeddings", bool) if d.get("tie_word_embeddings") is not None else False,
            bos_token_id=bos,
            eos_token_ids=_token_ids(d, "eos_token_id"),
            torch_dtype=str(d.get("torch_dtype", "bfloat16")),
            architecture=str(arch),
            extra={k: v for k, v in d.items() if k not in known},
        )
        cfg.validate()
        return cfg

    @staticmethod
    def from_folder(folder: str) -> "LlamaConfig":
        path = os.path.join(folder, "config.json")
        try:
            with open(path) as f:
                d = json.load(f)
        except FileNotFoundError:
            raise ConfigError(f"{path} not found: a model folder holds config.json and model.safetensors") from None
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path} is not valid JSON: {e}") from None
        return LlamaConfig.from_dict(d)

    def validate(self):
        for key in ("hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                    "num_key_value_heads", "head_dim", "vocab_size", "max_position_embeddings"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"config.json: '{key}' must be positive, got {getattr(self, key)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(f"config.json: 'num_attention_heads' {self.num_attention_heads} is not a multiple "
                              f"of 'num_key_value_heads' {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"config.json: 'head_dim' {self.head_dim} must be even (rotary pairs)")
        if not self.rms_norm_eps > 0:
            raise ConfigError("config.json: 'rms_norm_eps' must be positive")
        if not self.rope_theta > 0:
            raise ConfigError("config.json: 'rope_theta' must be positive")
        s = self.rope_scaling
        if s is not None:
            if s.factor <= 0 or s.original_max_position_embeddings <= 0:
                raise ConfigError("config.json: rope_scaling factor and original_max_position_embeddings must be positive")
            if s.high_freq_factor == s.low_freq_factor:
                raise ConfigError("config.json: rope_scaling high_freq_factor must differ from low_freq_factor")
        for t in self.eos_token_ids + ((self.bos_token_id,) if self.bos_token_id is not None else ()):
            if not 0 <= t < self.vocab_size:
                raise ConfigError(f"config.json: token id {t} is outside the vocabulary of {self.vocab_size}")

    def to_dict(self) -> dict:
        d = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": None,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "attention_bias": False,
            "mlp_bias": False,
            "torch_dtype": self.torch_dtype,
        }
        if self.rope_scaling is not None:
            s = self.rope_scaling
            d["rope_scaling"] = {"rope_type": "llama3", "factor": s.factor, "low_freq_factor": s.low_freq_factor,
                                 "high_freq_factor": s.high_freq_factor,
                                 "original_max_position_embeddings": s.original_max_position_embeddings}
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        return d
