"""Choice of the next token from float32 logits.

The reference picks ``argmax`` when the temperature is 0 and otherwise draws from
``softmax(logits / temperature)`` cut to the top-p nucleus (crates/burn-lm-llama/src/server/
llama3.rs:454-462, generation/generate.rs:87-91, generation/sampling.rs:9-71), with a seeded
generator and "seed 0 = a fresh seed for each request".  Here both run as HIP kernels on the
whole batch; the random number of a draw depends only on (seed, request, index of the token in
that request), so a request samples the same tokens whatever else is in its batch."""
from __future__ import annotations

import os
from typing import List, Sequence

import torch

_MASK = (1 << 64) - 1
UNIFORM_RING = 8


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def uniform(seed: int, request: int, index: int) -> float:
    """Counter-based uniform number in [0, 1) with 24 bits, a pure function of its arguments."""
    x = _splitmix64(seed & _MASK)
    x = _splitmix64(x ^ ((request + 1) * 0xD1B54A32D192ED03 & _MASK))
    x = _splitmix64(x ^ ((index + 1) * 0x8CB92BA72F3D8DD7 & _MASK))
    return (x >> 40) / float(1 << 24)


class Picked:
    """The tokens picked for the rows of one step.  ``device`` (int32 [rows], on the GPU) can feed
    the next step without the host having seen the tokens; ``tokens()`` waits for their copy to
    the host, which was started when they were picked, and returns them as a list."""

    def __init__(self, device_tokens: torch.Tensor):
        self.device = device_tokens
        self._host = torch.empty(device_tokens.shape, dtype=device_tokens.dtype, pin_memory=True)
        self._host.copy_(device_tokens, non_blocking=True)
        self._done = torch.cuda.Event()
        self._done.record()

    def tokens(self) -> List[int]:
        self._done.synchronize()
        return self._host.tolist()


class Sampler:
    """temperature == 0: greedy, lowest index wins ties.  temperature > 0: temperature softmax,
    nucleus of mass top_p (1.0 keeps everything), inverse-CDF draw."""

    def __init__(self, temperature: float = 0.0, top_p: float = 0.9, seed: int = 0, ops=None):
        if temperature < 0:
            raise ValueError(f"temperature must be >= 0, got {temperature}")
        if not 0 < top_p <= 1:
            raise ValueError(f"top_p must be in (0, 1], got {top_p}")
        self.temperature, self.top_p = float(temperature), float(top_p)
        # seed 0 means a fresh random seed (crates/burn-lm-llama/src/server/llama3.rs:454-457)
        self.seed = int(seed) if seed else int.from_bytes(os.urandom(8), "little")
        self._ops = ops
        self._ring, self._next = [], 0

    def _pinned_uniforms(self, requests, indices):
        """The uniforms of one step in pinned host memory that the kernel reads in place: no copy is
        queued and no pinned buffer is allocated per step.  A ring of buffers; one is written again
        only after the kernel that read it has run.  The numbers are written by the native core
        (blm_uniforms: the same function as ``uniform`` above)."""
        n = len(requests)
        if len(self._ring) < UNIFORM_RING:
            self._ring.append([torch.empty(max(n, 64), dtype=torch.float32).pin_memory(), None])
            slot = self._ring[-1]
        else:
            slot = self._ring[self._next % UNIFORM_RING]
            self._next += 1
        if slot[1] is not None:
            slot[1].synchronize()     # the kernel that read this buffer last has run (long since, as a rule)
        if slot[0].numel() < n:
            slot[0] = torch.empty(n, dtype=torch.float32).pin_memory()
        from ..cache import core as _core
        _core.library().blm_uniforms(self.seed & _MASK, n, _core.ints(list(requests)), _core.ints(list(indices)),
                                     slot[0].data_ptr())
        return slot

    @property
    def greedy(self):
        return self.temperature == 0.0

    def uniforms(self, requests: Sequence[int], indices: Sequence[int]) -> List[float]:
        return [uniform(self.seed, r, i) for r, i in zip(requests, indices)]

    def pick_device(self, logits: torch.Tensor, requests: Sequence[int], indices: Sequence[int]) -> Picked:
        """logits float32 [rows, vocab] on the GPU -> one token per row, left on the GPU; nothing here
        waits for the GPU."""
        ops = self._ops
        if ops is None:
            from ..csrc import ops
            self._ops = ops
        if self.greedy:
            out = ops.argmax(logits)
        else:
            slot = self._pinned_uniforms(requests, indices)
            out = ops.sample(logits, slot[0][:logits.shape[0]], self.temperature, self.top_p)
            slot[1] = torch.cuda.Event()
            slot[1].record()
        return Picked(out)

    def pick(self, logits: torch.Tensor, requests: Sequence[int], indices: Sequence[int]) -> List[int]:
        """logits float32 [rows, vocab] on the GPU -> one token per row, as host integers."""
        return self.pick_device(logits, requests, indices).tokens()
