"""Loads the tensors a model asks for, by name, from a model folder.

Floating tensors are kept as the checkpoint stores them, in bfloat16 (half precision is
converted to it), and a tensor stored in 32 bits stays in 32 bits; a float32 run widens all of
them (exactly).  Integer tables become int32.  All problems of a checkpoint come back in one
error: tensors the model needs but the folder lacks, tensors the folder holds but the model does
not know, and tensors whose shape is wrong.  (The reference reports a load failure as one string,
crates/burn-lm-llama/src/nn/llama/base.rs:157-158, and unwraps it in the server,
server/llama3.rs:526-543.)"""
from __future__ import annotations

import re
from typing import Dict, Sequence

import torch

from ..parts.base import TensorSpec
from . import safetensors_io as st


class WeightError(ValueError):
    def __init__(self, folder, missing, unexpected, wrong_shape, wrong_kind):
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.wrong_shape, self.wrong_kind = list(wrong_shape), list(wrong_kind)
        lines = [f"checkpoint in {folder} does not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, got, want in self.wrong_shape:
            lines.append(f"  wrong shape: {name} is {list(got)}, the model needs {list(want)}")
        for name, got, want in self.wrong_kind:
            lines.append(f"  wrong dtype: {name} is {got}, the model needs {want} data")
        super().__init__("\n".join(lines))


def _is_float(dt):
    return dt in (torch.float32, torch.bfloat16, torch.float16, torch.float64)


def check(folder, available: Dict[str, st.SafetensorsFile], specs: Dict[str, TensorSpec],
          ignorable: Sequence[str] = ()):
    pats = [re.compile(p) for p in ignorable]
    missing = [n for n in specs if n not in available]
    unexpected = [n for n in available if n not in specs and not any(p.match(n) for p in pats)]
    wrong_shape, wrong_kind = [], []
    for n, spec in specs.items():
        if n not in available:
            continue
        f = available[n]
        if tuple(f.shape(n)) != tuple(spec.shape):
            wrong_shape.append((n, f.shape(n), spec.shape))
        if (spec.kind == "float") != _is_float(f.dtype(n)):
            wrong_kind.append((n, str(f.dtype(n)).replace("torch.", ""), "floating-point" if spec.kind == "float" else "integer"))
    if missing or unexpected or wrong_shape or wrong_kind:
        raise WeightError(folder, sorted(missing), sorted(unexpected), wrong_shape, wrong_kind)


def stored_dtype_to_kept(stored: torch.dtype, kind: str, run_dtype: torch.dtype) -> torch.dtype:
    if kind == "int":
        return torch.int32
    if run_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32
    return torch.bfloat16


def load(folder: str, specs: Dict[str, TensorSpec], run_dtype: torch.dtype, device,
         ignorable: Sequence[str] = (), available=None) -> Dict[str, torch.Tensor]:
    available = available if available is not None else st.open_folder(folder)
    check(folder, available, specs, ignorable)
    out = {}
    for name, spec in specs.items():
        f = available[name]
        t = f.tensor(name)
        out[name] = t.to(device=device, dtype=stored_dtype_to_kept(t.dtype, spec.kind, run_dtype), copy=True).contiguous()
    for f in {id(f): f for f in available.values()}.values():
        f.close()
    return out
