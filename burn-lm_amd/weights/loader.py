"""Loads the tensors a model asks for, by name, from a model folder.

Floating tensors are kept in bfloat16 (float16 is rounded to it: three bits of its fraction go),
and a tensor stored in 32 bits stays in 32 bits (``cast_32bit`` rounds such matrices to bfloat16 as
well, as the reference casts what it reads to its backend's type,
crates/burn-lm-llama/src/nn/llama/base.rs:155-177); a float32 run widens all of them (exactly).
Integer tables become int32.  All problems of a checkpoint come back in one
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
        lines = [f"{folder} does not fit the model:"]
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


def check(where, available: Dict[str, tuple], specs: Dict[str, TensorSpec], ignorable: Sequence[str] = ()):
    """available: name -> (shape, dtype) of what a checkpoint (a folder, or tensors in memory) holds."""
    pats = [re.compile(p) for p in ignorable]
    missing = [n for n in specs if n not in available]
    unexpected = [n for n in available if n not in specs and not any(p.match(n) for p in pats)]
    wrong_shape, wrong_kind = [], []
    for n, spec in specs.items():
        if n not in available:
            continue
        shape, dtype = available[n]
        if tuple(shape) != tuple(spec.shape):
            wrong_shape.append((n, shape, spec.shape))
        if (spec.kind == "float") != _is_float(dtype):
            wrong_kind.append((n, str(dtype).replace("torch.", ""), "floating-point" if spec.kind == "float" else "integer"))
    if missing or unexpected or wrong_shape or wrong_kind:
        raise WeightError(where, sorted(missing), sorted(unexpected), wrong_shape, wrong_kind)


def stored_dtype_to_kept(stored: torch.dtype, kind: str, run_dtype: torch.dtype, cast_32bit: bool = False,
                         dims: int = 1) -> torch.dtype:
    """Integer tables: int32.  A float32 run: float32 (exact for every stored type).  A bfloat16 run:
    bfloat16, float16 rounded to it (three bits of its fraction go; its range is the narrower one, so
    nothing overflows); a tensor stored in 32 bits stays in 32 bits, unless cast_32bit asks for
    matrices (two and more dimensions) in the run's type as well."""
    if kind == "int":
        return torch.int32
    if run_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.bfloat16 if cast_32bit and dims >= 2 else torch.float32
    return torch.bfloat16


def place(where, tensors: Dict[str, torch.Tensor], specs: Dict[str, TensorSpec], run_dtype: torch.dtype, device,
          ignorable: Sequence[str] = (), cast_32bit: bool = False) -> Dict[str, torch.Tensor]:
    """The same as load() for tensors that are in memory already (the random-weights mode that
    writes no file): checked against the model's wishes, moved and kept by the same rules."""
    check(where, {n: (tuple(t.shape), t.dtype) for n, t in tensors.items()}, specs, ignorable)
    out = {}
    for name, spec in specs.items():
        t = tensors[name]
        kept = stored_dtype_to_kept(t.dtype, spec.kind, run_dtype, cast_32bit, t.dim())
        out[name] = t.to(device=device, dtype=kept).contiguous()
    return out


def load(folder: str, specs: Dict[str, TensorSpec], run_dtype: torch.dtype, device,
         ignorable: Sequence[str] = (), available=None, cast_32bit: bool = False) -> Dict[str, torch.Tensor]:
    available = available if available is not None else st.open_folder(folder)
    check(f"checkpoint in {folder}", {n: (tuple(f.shape(n)), f.dtype(n)) for n, f in available.items()}, specs, ignorable)
    out = {}
    for name, spec in specs.items():
        f = available[name]
        t = f.tensor(name)
        kept = stored_dtype_to_kept(t.dtype, spec.kind, run_dtype, cast_32bit, t.dim())
        out[name] = t.to(device=device, dtype=kept, copy=True).contiguous()
    for f in {id(f): f for f in available.values()}.values():
        f.close()
    return out


def kept_wide(tensors: Dict[str, torch.Tensor], run_dtype: torch.dtype):
    """Names of the matrices that stayed in 32 bits in a run of a narrower type: products with them
    run on the float32 kernels (exact, slower, twice the memory)."""
    if run_dtype == torch.float32:
        return []
    return [n for n, t in tensors.items() if t.dim() >= 2 and t.dtype == torch.float32]
