"""Dense SwiGLU feed-forward: ``(silu(x W1) * (x W3)) W2`` without bias
(crates/burn-lm-llama/src/nn/fftn.rs:44-46; W1 = gate, W3 = up, W2 = down,
nn/llama/import.rs:22-31).  Gate and up run as one product on the stacked weight; silu and the
product are float32, in the product's own epilogue when few rows run (decode) and in a kernel of
their own otherwise."""
from __future__ import annotations

import torch

from .base import FeedForward, TensorSpec


class SwiGLU(FeedForward):
    """params: width, inner.  names: gate, up, down."""
    graph_safe = True


    def tensor_specs(self):
        d, i = self.params["width"], self.params["inner"]
        return {self.names["gate"]: TensorSpec((i, d)), self.names["up"]: TensorSpec((i, d)),
                self.names["down"]: TensorSpec((d, i))}

    def bind(self, tensors, rt):
        self.rt = rt
        g, u = tensors[self.names["gate"]], tensors[self.names["up"]]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        self.w_gate_up = rt.weight(torch.cat([g, u], dim=0), gated=True)
        self.w_down = rt.weight(tensors[self.names["down"]])
        self.inner = self.params["inner"]

    def step_bytes(self, rows):
        return sum(w.w.numel() * w.w.element_size() for w in (self.w_gate_up, self.w_down))

    def step_flops(self, rows):
        return 2 * rows * (self.w_gate_up.w.numel() + self.w_down.w.numel())

    def forward(self, x, step):
        rt = self.rt
        return rt.linear(rt.gated_linear(x, self.w_gate_up), self.w_down, partials=True)
