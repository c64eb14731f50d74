"""Arrangements of a layer's parts.

``pre_norm``: ``h = x + mixer(norm1(x)); y = h + ffn(norm2(h))``
(crates/burn-lm-llama/src/nn/transformer.rs:241-256).  Each add happens inside the next norm's
kernel on the float32 residual stream, so a block takes the pending ``delta`` of the block
before it and hands on its own."""
from __future__ import annotations

from .base import Block


class PreNormBlock(Block):
    roles = {"mixer_norm": "norm", "mixer": "mixer", "ffn_norm": "norm", "feed_forward": "feed_forward"}

    def forward(self, h, delta, step, view):
        x = self.mixer_norm.add_norm(h, delta)
        a = self.mixer.forward(x, step, view)
        return self.feed_forward.forward_after_norm(h, a, self.ffn_norm, step)
