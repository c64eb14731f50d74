"""RMS norm with the residual add fused in front of it.

``y = x / sqrt(mean(x^2) + eps) * gamma`` (crates/burn-lm-llama/src/nn/transformer.rs:60-62,
vector at :278-297).  The sum of squares, the root and the scaling are float32; the add that
precedes the norm in a block (transformer.rs:248-255) is done here, on the float32 residual.
"""
from __future__ import annotations

import torch

from .base import Norm, TensorSpec


class RMSNorm(Norm):
    """params: width, eps.  names: weight."""
    graph_safe = True


    def tensor_specs(self):
        return {self.names["weight"]: TensorSpec((self.params["width"],))}

    def bind(self, tensors, rt):
        self.rt = rt
        self.gamma = tensors[self.names["weight"]].contiguous()
        self.eps = float(self.params["eps"])

    def step_bytes(self, rows):
        return self.gamma.numel() * self.gamma.element_size()

    def rms_constants(self):
        return self.gamma, self.eps

    def add_norm(self, h, delta, rows=None, write_h=True):
        n = h.shape[0] if rows is None else rows.shape[0]
        out = torch.empty(n, h.shape[1], dtype=self.rt.dtype, device=h.device)
        return self.rt.ops.add_rmsnorm(h, delta, self.gamma, self.eps, out, rows=rows, write_h=write_h)
