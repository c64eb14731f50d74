"""Rotary position encoding with optional llama3 frequency scaling.

Angles: ``theta_i = theta^(-2i/head_dim)``, scaled "by parts" as in
crates/burn-lm-llama/src/nn/pos_encoding.rs:107-138; a token at absolute position p has its
pairs turned by ``p * theta_i`` (pos_encoding.rs:66-79, vector :165-174).  The table of cosines
and sines is computed once in float64 on the host and kept in float32; the rotation itself is
float32 in the kernel, rounded once.

Pairing: the reference pairs adjacent lanes ``(2i, 2i+1)`` and permutes Hugging Face q/k rows
into that order when it imports them (nn/llama/import.rs:94-127).  ``pairing="half"`` pairs
``(i, i + head_dim/2)`` instead, which is the same function on un-permuted Hugging Face rows,
so such checkpoints load without a re-layout.

``rotary_dim`` (default: all of head_dim) turns only the first that many lanes of every head, with
``theta_i = theta^(-2i/rotary_dim)``, and passes the rest through: the table holds angle zero for
their pairs, so the kernels need not know (pairs of "half" are then ``(i, i + rotary_dim/2)``).
"""
from __future__ import annotations

import math

import numpy as np
import torch

from .base import PositionEncoding

PAIRING = {"interleaved": 0, "half": 1}


def rope_frequencies(head_dim, theta, scaling=None, rotary_dim=None):
    """float64 [head_dim/2].  scaling: None or (factor, low_freq_factor, high_freq_factor, old_context).
    rotary_dim: lanes of a head that turn (default all); the pairs beyond them get frequency zero."""
    turning = head_dim if rotary_dim is None else int(rotary_dim)
    i = np.arange(0, turning, 2, dtype=np.float64)
    f = np.power(float(theta), -i / turning)
    if scaling is not None:
        factor, low, high, old = (float(v) for v in scaling)
        wavelen = 2.0 * math.pi / f
        smooth = (old / wavelen - low) / (high - low)
        mid = (1.0 - smooth) * f / factor + smooth * f
        f = np.where(wavelen < old / high, f, np.where(wavelen > old / low, f / factor, mid))
    if turning < head_dim:
        f = np.concatenate([f, np.zeros((head_dim - turning) // 2)])
    return f


class RotaryEncoding(PositionEncoding):
    """params: head_dim, theta, scaling (None or 4 numbers), pairing ("half" | "interleaved"),
    rotary_dim (optional: the lanes of a head that turn, an even number up to head_dim)."""
    graph_safe = True


    def bind(self, tensors, rt):
        self.rt = rt
        self.head_dim = int(self.params["head_dim"])
        if self.params["pairing"] not in PAIRING:
            raise ValueError(f"rotary pairing {self.params['pairing']!r} unknown; one of {list(PAIRING)}")
        self.pairing = PAIRING[self.params["pairing"]]
        self.rotary_dim = int(self.params.get("rotary_dim") or self.head_dim)
        if self.rotary_dim % 2 or not 2 <= self.rotary_dim <= self.head_dim or self.head_dim % 2:
            raise ValueError(f"rotary_dim must be an even number from 2 to head_dim = {self.head_dim}, got {self.rotary_dim}")
        self.freqs = rope_frequencies(self.head_dim, self.params["theta"], self.params.get("scaling"), self.rotary_dim)
        self._shared = {"table": None, "n_positions": 0}    # one table for this encoding and its adjacent-pair twin
        self._twin = None

    table = property(lambda self: self._shared["table"])
    n_positions = property(lambda self: self._shared["n_positions"])

    def prepare(self, n_positions, rt):
        ang = np.arange(n_positions, dtype=np.float64)[:, None] * self.freqs[None, :]
        cs = np.stack([np.cos(ang), np.sin(ang)], axis=-1).astype(np.float32)
        self._shared["table"] = torch.from_numpy(cs).to(rt.device)
        self._shared["n_positions"] = n_positions

    def for_projection(self, w_q, w_k, heads, kv_heads):
        """Pairs half a head apart are the same function as adjacent pairs on rows that are permuted
        within every head (row ``r * head_dim/2 + i`` goes to ``2i + r``), which is the re-layout the
        reference applies to such checkpoints (nn/llama/import.rs:99-126).  The kernels prefer
        adjacent pairs (both partners in one 16-column tile), so the projection's rows are permuted
        when they are bound and a twin of this encoding with adjacent pairs, sharing its table, does
        the rotating.  Keys are cached in the permuted lane order; the scores do not change, since
        queries are permuted alike."""
        if self.pairing == PAIRING["interleaved"]:
            return w_q, w_k, self
        if self._twin is None:
            twin = RotaryEncoding(dict(self.params, pairing="interleaved"), self.names)
            twin.bind({}, self.rt)
            twin._shared = self._shared
            self._twin = twin
        hd, rd = self.head_dim, self.rotary_dim

        def permute(w, n):
            heads = w.reshape(n, hd, w.shape[1])
            turning = heads[:, :rd].reshape(n, 2, rd // 2, w.shape[1]).transpose(1, 2).reshape(n, rd, w.shape[1])
            return torch.cat([turning, heads[:, rd:]], dim=1).reshape(n * hd, w.shape[1]).contiguous()

        return permute(w_q, heads), permute(w_k, kv_heads), self._twin

    def _check_pairs(self):
        if self.pairing == PAIRING["half"] and self.rotary_dim < self.head_dim:
            raise ValueError("pairs half the turning lanes apart exist only as adjacent pairs on permuted rows: "
                             "bind the projections through for_projection and use the encoding it hands back")

    def encode_and_store(self, qkv, step, view, heads, kv_heads, head_dim, store=True):
        self._check_pairs()
        if step.max_position >= self.n_positions:
            raise ValueError(f"position {step.max_position} is past the rotary table of {self.n_positions}")
        self.rt.ops.rope_kv_write(qkv, step.positions, step.token_seq, view.block_table(step), self.table,
                                  view.k, view.v, view.page_size, heads, kv_heads, head_dim, self.pairing,
                                  write_kv=store)

    def project_encode_store(self, x, w_qkv, step, view, heads, kv_heads, head_dim):
        """Projection, rotation and cache write in one kernel (the rotation applied to the float
        accumulators) where the runtime has a fused geometry for these sizes and this encoding's kernel
        exists for it; otherwise the three steps apart.  Which geometry suits which sizes is the
        runtime's answer (Runtime.qkv_plan); what is checked here is only what the rotation itself needs."""
        rt = self.rt
        self._check_pairs()
        M, K = x.shape
        n_qkv = (heads + 2 * kv_heads) * head_dim
        plan = rt.qkv_plan(M, n_qkv, K) if hasattr(rt, "qkv_plan") else None
        bf16 = x.dtype == view.k.dtype == torch.bfloat16 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
        raw, packable = getattr(w_qkv, "w", None), getattr(w_qkv, "packable", False)
        fused = None
        if (plan is not None and plan.kernel == "rows" and bf16 and self.pairing == PAIRING["interleaved"]
                and raw is not None and raw.dtype == torch.bfloat16 and raw.is_contiguous()
                and head_dim % 2 == 0 and K % 8 == 0 and x.stride(1) == 1):
            fused = "rows"
        elif (plan is not None and M <= 64 and bf16 and packable and not getattr(w_qkv, "gated", False)
                and rt.ops.gemv_qkv_rope_supported(M, K, head_dim, self.pairing)):
            fused = "packed"     # also where the row-ring kernel was the plan and this encoding has none for it
        if fused is None:
            return super().project_encode_store(x, w_qkv, step, view, heads, kv_heads, head_dim)
        if step.max_position >= self.n_positions:
            raise ValueError(f"position {step.max_position} is past the rotary table of {self.n_positions}")
        qkv = torch.empty(M, n_qkv, dtype=torch.bfloat16, device=x.device)
        if fused == "rows":
            return rt.ops.gemm_rows_qkv_rope(x, raw, qkv, step.positions, step.token_seq, view.block_table(step), self.table,
                                             view.k, view.v, view.page_size, heads, kv_heads, head_dim, write_kv=view.store,
                                             columns=plan.columns, rows=plan.rows)
        return rt.ops.gemv_qkv_rope(x, w_qkv.packed, qkv, step.positions, step.token_seq, view.block_table(step),
                                    self.table, view.k, view.v, view.page_size, heads, kv_heads, head_dim,
                                    self.pairing, write_kv=view.store)
