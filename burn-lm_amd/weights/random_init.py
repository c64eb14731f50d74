"""Random-weights mode: writes a model folder (config.json, model.safetensors) from a
configuration and a seed.  Matrices are N(0, std); norm weights are 1, or 1 + N(0, norm_jitter)
when a test wants a wrong norm mapping to show.  The reference's random start is burn's default
initialisers (crates/burn-lm-llama/src/nn/transformer.rs:45-73); its tests overwrite them with a
fixture (crates/burn-lm-llama/src/lib.rs:26-214)."""
from __future__ import annotations

import json
import os

import torch

from .. import registry
from . import safetensors_io as st


def random_tensors(arch, cfg, seed: int, std: float = 0.02, norm_jitter: float = 0.0,
                   dtype=torch.bfloat16, device="cpu"):
    """Yields (name, tensor) in checkpoint order; every tensor has a generator of its own, keyed
    by the seed and its index, so the values do not depend on what was drawn before."""
    for idx, (name, (shape, role)) in enumerate(arch.checkpoint_tensors(cfg).items()):
        g = torch.Generator(device=device)
        g.manual_seed((int(seed) * 1000003 + idx) & 0x7FFFFFFFFFFFFFFF)
        if role == "norm":
            t = torch.ones(shape, dtype=torch.float32, device=device)
            if norm_jitter:
                t = t + norm_jitter * torch.randn(shape, generator=g, dtype=torch.float32, device=device)
        else:
            t = torch.randn(shape, generator=g, dtype=torch.float32, device=device) * std
        yield name, t.to(dtype)


def write_model_folder(folder: str, config: dict, seed: int = 0, std: float = 0.02, norm_jitter: float = 0.0,
                       dtype=torch.bfloat16) -> str:
    """config: the contents of config.json (it names the architecture).  Returns the folder."""
    arch = registry.architecture_of(config)
    cfg = arch.read_config(config)
    os.makedirs(folder, exist_ok=True)
    out = dict(config)
    out["torch_dtype"] = str(dtype).replace("torch.", "")
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(out, f, indent=2)
    st.write_file(os.path.join(folder, "model.safetensors"),
                  random_tensors(arch, cfg, seed, std, norm_jitter, dtype),
                  metadata={"format": "pt", "seed": seed})
    return folder
