"""Token embedding and output head.

``h = table[ids]`` with no scaling (crates/burn-lm-llama/src/nn/transformer.rs:95) into the
float32 residual stream; ``logits = x W_out^T`` without bias in float32 (transformer.rs:102).
A tied head uses the embedding table itself: the ``[vocab, width]`` table is the head's
``[d_out, d_in]`` matrix (the reference leaves tying as a TODO, transformer.rs:82-84)."""
from __future__ import annotations

import torch

from .base import Part, TensorSpec


class Embedding(Part):
    """params: vocab, width.  names: weight."""
    graph_safe = True

    def tensor_specs(self):
        return {self.names["weight"]: TensorSpec((self.params["vocab"], self.params["width"]))}

    def bind(self, tensors, rt):
        self.rt = rt
        self.table = tensors[self.names["weight"]].contiguous()

    def step_bytes(self, rows):
        return rows * self.params["width"] * self.table.element_size()      # the rows that are looked up

    def forward(self, ids):
        h = torch.empty(ids.shape[0], self.params["width"], dtype=torch.float32, device=ids.device)
        return self.rt.ops.embed_gather(self.table, ids, h)

    def forward_from(self, ids, source_rows, source_cell):
        """The same where some tokens are still on the device: row t is element source_rows[t] of the
        array whose address is in source_cell, where source_rows[t] >= 0.  An embedding without this
        method gets its tokens gathered by a separate launch before the step."""
        h = torch.empty(ids.shape[0], self.params["width"], dtype=torch.float32, device=ids.device)
        return self.rt.ops.embed_gather_from(self.table, ids, source_rows, source_cell, h)


class LMHead(Part):
    """params: vocab, width.  names: weight (the embedding's name when tied)."""
    graph_safe = True

    def tensor_specs(self):
        return {self.names["weight"]: TensorSpec((self.params["vocab"], self.params["width"]))}

    def bind(self, tensors, rt):
        self.rt = rt
        self.weight = rt.weight(tensors[self.names["weight"]])

    def step_bytes(self, rows):
        return self.weight.w.numel() * self.weight.w.element_size() if rows else 0

    def step_flops(self, rows):
        return 2 * rows * self.weight.w.numel()

    def forward(self, x):
        return self.rt.linear(x, self.weight, out_dtype=torch.float32)
