"""Random-weights mode: writes a model folder (config.json, model.safetensors) from a
configuration and a seed, or hands the same tensors to an engine without the trip through a file.

Every value is a pure function of (seed, tensor name, index of the element in the tensor), computed
with 64-bit integer arithmetic alone up to one final float multiplication, so a tensor has the same
bytes whether it is made on the CPU or on the GPU, whole or in pieces, and whatever was made before
it.  Matrices are N(0, std) (the sum of twelve 16-bit uniform numbers, shifted and scaled: normal
to within what a weight initialisation can tell, exact in integers); norm weights are 1, or
1 + N(0, norm_jitter) when a test wants a wrong norm mapping to show.  ``Range(lo, hi)`` is the
fixture of the reference's tests (crates/burn-lm-llama/src/lib.rs:142-148: ``arange(n) * (hi - lo)
/ n + lo``), laid over a linear weight in the reference's ``[d_in, d_out]`` element order.  The
reference's own random start is burn's default initialisers
(crates/burn-lm-llama/src/nn/transformer.rs:45-73).

An architecture's ``checkpoint_tensors(config)`` gives ``{name: (shape, init)}``; ``init`` is one of
the initialisers below or a role name: ``"matrix"`` (a linear weight ``[d_out, d_in]``: Normal),
``"table"`` (an embedding table: Normal), ``"norm"`` (Ones)."""
from __future__ import annotations

import hashlib
import json
import os
from dataclasses import dataclass
from typing import Optional

import torch

from .. import registry
from . import safetensors_io as st

_GOLDEN = 0x9E3779B97F4A7C15
_M1, _M2 = 0xBF58476D1CE4E5B9, 0x94D049BB133111EB
CHUNK = {"cpu": 1 << 18, "cuda": 1 << 24}     # elements made at a time (the CPU's caches hold the smaller run)


def _s64(x: int) -> int:
    """The 64-bit pattern x as the signed integer torch's int64 holds."""
    x &= (1 << 64) - 1
    return x - (1 << 64) if x >= (1 << 63) else x


def _lsr(x, n):
    """Logical shift right of int64 values (torch's >> keeps the sign)."""
    return (x >> n) & ((1 << (64 - n)) - 1)


def _mix(x):
    """The finaliser of splitmix64 on int64 tensors (multiplications wrap)."""
    x = (x ^ _lsr(x, 30)) * _s64(_M1)
    x = (x ^ _lsr(x, 27)) * _s64(_M2)
    return x ^ _lsr(x, 31)


def tensor_key(seed: int, name: str) -> int:
    """64 bits from the seed and the tensor's name."""
    h = hashlib.sha256(f"{int(seed)}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little")


def standard_normal(key: int, start: int, count: int, device="cpu") -> torch.Tensor:
    """float32 [count]: elements start .. start+count-1 of the stream that belongs to key.  Element i
    takes the counters 4i, 4i+1, 4i+2; each gives 64 bits, whose twelve 16-bit fields are summed
    (mean 6 * 65535, variance 65536^2 - 1)."""
    i = torch.arange(start, start + count, dtype=torch.int64, device=device) * 4
    total = torch.zeros(count, dtype=torch.int64, device=device)
    for k in range(3):
        bits = _mix((i + k) * _s64(_GOLDEN) + _s64(key))
        for f in range(4):
            total += _lsr(bits, 16 * f) & 0xFFFF
    return (total - 6 * 65535).to(torch.float32) * (1.0 / 65536.0)


def uniform_integers(key: int, start: int, count: int, n: int, device="cpu") -> torch.Tensor:
    """int64 [count] in [0, n)."""
    i = torch.arange(start, start + count, dtype=torch.int64, device=device) * 4
    return _lsr(_mix(i * _s64(_GOLDEN) + _s64(key)), 1) % int(n)


@dataclass(frozen=True)
class Normal:
    """N(0, std); std None = the std the caller of the random mode asks for."""
    std: Optional[float] = None
    layout: str = "matrix"   # "matrix": a linear weight [d_out, d_in]; "table": rows of an embedding


@dataclass(frozen=True)
class Ones:
    """1 + N(0, jitter); jitter None = the caller's norm_jitter."""
    jitter: Optional[float] = None
    layout: str = "norm"


@dataclass(frozen=True)
class Range:
    """arange(n) * (hi - lo) / n + lo.  Over a linear weight the index runs in the reference's
    [d_in, d_out] order, so the checkpoint's [d_out, d_in] matrix holds the transposed ramp."""
    lo: float
    hi: float


@dataclass(frozen=True)
class IntegerTable:
    """Integers in [0, n), for tensors kept as int32 (routing tables and the like)."""
    n: int
    layout: str = "int"


ROLES = {"matrix": Normal(), "table": Normal(layout="table"), "norm": Ones()}


def _initialiser(init):
    if isinstance(init, str):
        try:
            return ROLES[init]
        except KeyError:
            raise ValueError(f"random weights: role {init!r} unknown; roles: {', '.join(ROLES)}") from None
    return init


def make_tensor(name, shape, init, seed, std=0.02, norm_jitter=0.0, dtype=torch.bfloat16, device="cpu",
                override=None, quick=False):
    """One tensor of a fresh checkpoint.  override: a Range that replaces the initialiser of every
    floating tensor (the reference's fixture), keeping the tensor's layout.  quick: normal deviates from the
    device's own generator in one launch per tensor instead of the counter-based stream (not reproducible
    across devices or in a folder; for runs under a profiler, where each of the stream's thousands of small
    launches is slow)."""
    init = _initialiser(init)
    shape = tuple(int(s) for s in shape)
    n = 1
    for s in shape:
        n *= s
    if isinstance(init, IntegerTable):
        key = tensor_key(seed, name)
        chunk = CHUNK[torch.device(device).type]
        parts = [uniform_integers(key, a, min(chunk, n - a), init.n, device) for a in range(0, n, chunk)]
        return torch.cat(parts).reshape(shape).to(torch.int32)
    layout = getattr(init, "layout", "matrix")
    if override is not None:
        init = override
    if isinstance(init, Range):
        ramp = torch.arange(n, dtype=torch.float64, device=device) * ((init.hi - init.lo) / n) + init.lo
        if layout == "matrix" and len(shape) == 2:
            ramp = ramp.reshape(shape[1], shape[0]).t()
        return ramp.reshape(shape).to(dtype).contiguous()
    key = tensor_key(seed, name)
    if isinstance(init, Ones):
        jitter = norm_jitter if init.jitter is None else init.jitter
        if not jitter:
            return torch.ones(shape, dtype=dtype, device=device)
        scale, offset = float(jitter), 1.0
    elif isinstance(init, Normal):
        scale, offset = float(std if init.std is None else init.std), 0.0
    else:
        raise ValueError(f"random weights: {name} has the initialiser {init!r}, which is none of "
                         f"Normal, Ones, Range, IntegerTable or a role name")
    if quick:
        g = torch.Generator(device=device)
        g.manual_seed(tensor_key(seed, name) & 0x7FFFFFFF)
        z = torch.randn(shape, dtype=torch.float32, device=device, generator=g) * scale
        return (z + offset if offset else z).to(dtype)
    out = torch.empty(n, dtype=dtype, device=device)
    chunk = CHUNK[torch.device(device).type]
    for a in range(0, n, chunk):
        c = min(chunk, n - a)
        z = standard_normal(key, a, c, device) * scale
        out[a:a + c] = (z + offset if offset else z).to(dtype)
    return out.reshape(shape)


def random_tensors(arch, cfg, seed: int, std: float = 0.02, norm_jitter: float = 0.0,
                   dtype=torch.bfloat16, device="cpu", init=None, names=None, quick=False):
    """Yields (name, tensor) in checkpoint order.  init: a Range for every floating tensor instead of
    the architecture's initialisers.  names: passed on to architectures that know several checkpoint
    layouts (the Llama architecture: "hf" or "meta")."""
    if arch.checkpoint_tensors is None:
        raise ValueError(f"architecture {arch.name} has no checkpoint_tensors: it cannot make random weights")
    table = arch.checkpoint_tensors(cfg) if names is None else arch.checkpoint_tensors(cfg, names=names)
    for name, (shape, how) in table.items():
        yield name, make_tensor(name, shape, how, seed, std, norm_jitter, dtype, device, override=init, quick=quick)


def write_model_folder(folder: str, config: dict, seed: int = 0, std: float = 0.02, norm_jitter: float = 0.0,
                       dtype=torch.bfloat16, init=None, names=None) -> str:
    """config: the contents of config.json (it names the architecture).  Returns the folder."""
    arch = registry.architecture_of(config)
    cfg = arch.read_config(config)
    os.makedirs(folder, exist_ok=True)
    out = dict(config)
    out["torch_dtype"] = str(dtype).replace("torch.", "")
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(out, f, indent=2)
    st.write_file(os.path.join(folder, "model.safetensors"),
                  random_tensors(arch, cfg, seed, std, norm_jitter, dtype, init=init, names=names),
                  metadata={"format": "pt", "seed": seed})
    return folder
