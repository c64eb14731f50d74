"""From a model folder to an engine: read config.json, find the architecture in the registry,
plan the parts, load the tensors by name, build the cache."""
from __future__ import annotations

import json
import os
import sys
import time

import torch

from .. import models, parts, registry  # noqa: F401  (registration happens at import)
from ..errors import ConfigError
from ..weights import loader, safetensors_io
from .engine import Engine
from .model import Model
from .runtime import Runtime

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "f32": torch.float32,
          "fp32": torch.float32}


def parse_dtype(name):
    if isinstance(name, torch.dtype):
        return name
    try:
        return DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"dtype {name!r} unknown; one of bfloat16, float32") from None


def read_config(folder):
    path = os.path.join(folder, "config.json")
    try:
        with open(path) as f:
            d = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"{path} not found: a model folder holds config.json and model.safetensors") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path} is not valid JSON: {e}") from None
    arch = registry.architecture_of(d)
    return arch, arch.read_config(d)


def _notice_wide(tensors, dtype, where):
    wide = loader.kept_wide(tensors, dtype)
    if wide:
        print(f"note: {len(wide)} matrices of {where} are stored in 32 bits and stay so in this bfloat16 run "
              f"(first: {wide[0]}): their products run on the float32 kernels, exact but slower and twice the "
              f"memory; cast_32bit=True (--cast-32bit) rounds them to bfloat16 when they are loaded", file=sys.stderr)


def load_model(folder, dtype="bfloat16", device="cuda:0", cast_32bit=False):
    """-> (Model bound to its tensors, Runtime, typed configuration)."""
    dtype = parse_dtype(dtype)
    arch, cfg = read_config(folder)
    rt = Runtime(dtype=dtype, device=device)
    available = safetensors_io.open_folder(folder)
    plan = arch.plan(cfg, set(available))
    model = Model(plan)
    tensors = loader.load(folder, model.tensor_specs(), dtype, rt.device, plan.ignorable_tensors, available, cast_32bit)
    _notice_wide(tensors, dtype, folder)
    model.bind(tensors, rt)
    model.config = cfg
    model.architecture = arch
    return model, rt, cfg


def _engine(model, rt, cfg, max_tokens, max_seqs, max_context, page_size, graphs):
    eng = Engine(model, rt, max_tokens=max_tokens, max_seqs=max_seqs, max_context=max_context, page_size=page_size,
                 graphs=graphs)
    eng.config = cfg
    return eng


def load_engine(folder, dtype="bfloat16", max_tokens=8192, max_seqs=None, max_context=None, device="cuda:0",
                page_size=64, graphs=True, cast_32bit=False):
    t0 = time.time()
    model, rt, cfg = load_model(folder, dtype, device, cast_32bit)
    eng = _engine(model, rt, cfg, max_tokens, max_seqs, max_context, page_size, graphs)
    eng.load_seconds = time.time() - t0
    return eng


def random_engine(config: dict, seed=0, dtype="bfloat16", max_tokens=8192, max_seqs=None, max_context=None,
                  device="cuda:0", std=0.02, norm_jitter=0.0, page_size=64, graphs=True, stored_dtype=torch.bfloat16,
                  quick_weights=False):
    """Engine with seeded random weights made directly on the GPU: the very tensors that the
    random-weights mode writes into a folder for this configuration, seed and stored type (every
    value is a function of seed, tensor name and element index), checked and kept by the loader's
    rules, without the trip through a file."""
    from ..weights.random_init import random_tensors
    dtype = parse_dtype(dtype)
    arch = registry.architecture_of(config)
    cfg = arch.read_config(config)
    rt = Runtime(dtype=dtype, device=device)
    made = dict(random_tensors(arch, cfg, seed, std=std, norm_jitter=norm_jitter, dtype=stored_dtype, device=rt.device,
                               quick=quick_weights))
    plan = arch.plan(cfg, set(made))
    model = Model(plan)
    tensors = loader.place(f"the random checkpoint of {arch.name}", made, model.tensor_specs(), dtype, rt.device,
                           plan.ignorable_tensors)
    del made
    model.bind(tensors, rt)
    model.config, model.architecture = cfg, arch
    return _engine(model, rt, cfg, max_tokens, max_seqs, max_context, page_size, graphs)
