"""Grouped-query attention over the paged cache.

``q, k, v = x Wq, x Wk, x Wv`` without bias, heads split as ``feature j -> head j // head_dim``
(crates/burn-lm-llama/src/nn/attention/mha.rs:121-140); position encoding of q and k, append to
the cache (mha.rs:91-95); query head h reads key-value head ``h // (heads / kv_heads)``
(mha.rs:174-185); ``softmax(q k^T * scale + causal mask) v`` (mha.rs:143-171, scale
``1/sqrt(head_dim)`` at :159); output projection (mha.rs:118).  The three projections run as
one product on the stacked weight.
"""
from __future__ import annotations

import torch


from .base import KVNeed, Mixer, TensorSpec

# Blocks the decode attention aims for when it cuts the key ranges into pieces: one round of at most one
# block per compute unit, at least half of them busy, and no cutting from one block per unit on.
# (DECODE_TARGET_PER_UNIT is what the generic kernel's one-wavefront blocks aim for.)
DECODE_TARGET_PER_UNIT = 2
DECODE_MIN_PER_UNIT = 0.5
DECODE_MAX_PIECES = 32


def decode_splits(pages: int, blocks: int, head_dim: int, compute_units: int = 256) -> int:
    """Into how many pieces the decode attention cuts a sequence's pages.  Every piece is a block of
    four wavefronts that take pages in turn, and the pieces' results are merged by the last block to
    finish, so a piece should hold two pages per wavefront (eight), or down to two pages in all while
    that leaves fewer than half the compute units busy; and all blocks should run in one round, at most
    one per compute unit: a second, partial round costs more than longer pieces do (us per call at a
    context of 4,096, blocks in brackets; heads of 64, batch 6: 4 pieces (192) 13.8, 5 (240) 14.0, 6 (288)
    16.2, 8 (384) 14.9, 10 (480) 14.5; batch 10: 3 (240) 18.5, 4 (320) 21.2, 6 (480) 18.9, 7 (560) 21.5;
    batch 24: whole (192) 32.3, 3 (576) 41.6; heads of 128, whose blocks fill a compute unit's shared
    memory alone: batch 10: 3 (240) 32.8, 4 (320) 44.0; batch 20: whole (160) 54.0, 2 (320) 71.9; the
    same at contexts of 2,048 and 16,384).
    Measured at context 4096, head_dim 64, ms per step: batch 1: 16 pieces 0.870, 8: 0.880, 64: 1.002;
    batch 2: 8 pieces 0.909, 16: 0.928; batch 4: 8 pieces 0.961, 16: 0.988; batch 8: 4 and 8 pieces equal.
    Never more than DECODE_MAX_PIECES: at batch 1 and a context of 32,768 the kernel takes 18.6 us with
    32 pieces, 22.3 with 64 and 31.4 with 128 (every piece costs its look-ups, its partial result and
    its arrival; the merge reads them all).  And no cutting at all once every compute unit has a block:
    an uncut sequence needs no partial result, no arrival and no merge (batch 32, context 4096: 48.5 us
    uncut, 57.8 in two pieces; context 16,384: 171 against 186).  Nor for short ranges, two pages per
    wavefront and (for heads up to 64) three: a merge costs three trips through device-coherent memory in a
    row, about 3 us, a further page per wavefront about 2 (us per call, cut in two / uncut, 32 heads of 64
    in 8 groups: 8 pages at batch 1 7.1 / 6.6, at batch 8 8.1 / 7.0; 11 pages 7.9 / 8.0 and 9.0 / 8.4;
    16 pages, cut in four, 7.3 / 10.2; heads of 128: 8 pages 11.1 / 11.1, 11 pages 12.8 / 13.7).  Where a
    range is cut although the blocks are few, it is cut down to two pages per piece, not four (one
    compute unit brings a page of wide heads, 32 KB, no faster than 60 GB/s: heads of 128 at batch 1,
    11 pages: 2 pieces 13.0, uncut 11.1, 6 pieces 10.4; 16 pages: 4 pieces 12.1, 8 pieces 10.7; heads of 64,
    16 pages: 4 pieces 7.9, 8 pieces 7.3), and ranges of up to 16 pages stay whole from a block for every
    fourth compute unit on (heads of 128, 11 pages at batch 8: uncut 12.3, in two 14.0; 16 pages at batch
    16: 16.9 / 18.5; heads of 64, 16 pages at batch 8: 9.1 / 10.0)."""
    if blocks >= compute_units or pages <= (12 if head_dim <= 64 else 8):
        return 1
    if pages <= 16 and blocks * 4 >= compute_units:
        return 1
    least = max(1, int(compute_units * DECODE_MIN_PER_UNIT))
    n = min(max(1, pages // 8), max(1, compute_units // blocks), DECODE_MAX_PIECES)
    if blocks * n < least:
        n = max(n, min(max(1, pages // 2), (least + blocks - 1) // blocks, DECODE_MAX_PIECES))
    return max(1, n)


class Attention(Mixer):
    """params: width, heads, kv_heads, head_dim, scale, window (0 = all keys), position (the
    position-encoding object, given by the model builder).  names: q, k, v, o."""
    graph_safe = True


    def tensor_specs(self):
        p = self.params
        d, hd = p["width"], p["head_dim"]
        return {self.names["q"]: TensorSpec((p["heads"] * hd, d)),
                self.names["k"]: TensorSpec((p["kv_heads"] * hd, d)),
                self.names["v"]: TensorSpec((p["kv_heads"] * hd, d)),
                self.names["o"]: TensorSpec((d, p["heads"] * hd))}

    def cache_need(self):
        p = self.params
        return KVNeed(p["kv_heads"], p["head_dim"], int(p.get("window", 0)))

    def bind(self, tensors, rt):
        self.rt = rt
        p = self.params
        self.heads, self.kv_heads, self.head_dim = p["heads"], p["kv_heads"], p["head_dim"]
        self.scale = float(p["scale"])
        self.window = int(p.get("window", 0))
        ws = [tensors[self.names[r]] for r in ("q", "k", "v")]
        ws[0], ws[1], self.position = p["position"].for_projection(ws[0], ws[1], self.heads, self.kv_heads)
        if len({w.dtype for w in ws}) != 1:
            ws = [w.float() for w in ws]
        self.w_qkv = rt.weight(torch.cat(ws, dim=0))
        self.w_o = rt.weight(tensors[self.names["o"]])

    def step_bytes(self, rows):
        return sum(w.w.numel() * w.w.element_size() for w in (self.w_qkv, self.w_o))

    def step_flops(self, rows):
        return 2 * rows * (self.w_qkv.w.numel() + self.w_o.w.numel())

    def mixing_flops(self, past, new):
        """Scores and weighted values: 2 * 2 * heads * head_dim per (query, visible key) pair."""
        keys = sum(min(past + t + 1, self.window) if self.window else past + t + 1 for t in range(new)) if self.window \
            else new * past + new * (new + 1) // 2
        return 4 * self.heads * self.head_dim * keys

    def forward(self, x, step, view):
        if view.v.shape[1:3] != (self.kv_heads, self.head_dim):
            raise ValueError("the attention mixer needs values of the keys' head count and head size")
        return self.output(self.attend(self.project(x, step, view), step, view))

    def project(self, x, step, view):
        """q, k, v of the step's tokens, q and k encoded by position, k and v stored in the cache."""
        return self.position.project_encode_store(x, self.w_qkv, step, view, self.heads, self.kv_heads, self.head_dim)

    def output(self, attended):
        return self.rt.linear(attended, self.w_o, partials=True)   # the block's next norm sums partial products

    def attend(self, qkv, step, view):
        """Every token's queries over its sequence's cached keys and values -> [tokens, heads * head_dim]."""
        rt = self.rt
        nh, nkv, hd = self.heads, self.kv_heads, self.head_dim
        out = torch.empty(qkv.shape[0], nh * hd, dtype=rt.dtype, device=qkv.device)
        table = view.block_table(step)
        aligned = qkv.shape[1] % 8 == 0
        if step.max_new == 1 and aligned and rt.ops.attn_decode_supported(rt.dtype, hd, view.page_size):
            # decode: cut each sequence's keys so that the whole chip has work
            span = step.max_len_after if not self.window else min(step.max_len_after, self.window + view.page_size)
            pages = (span + view.page_size - 1) // view.page_size
            blocks = qkv.shape[0] * nkv * ((nh // nkv + 15) // 16)
            n_splits = decode_splits(pages, blocks, hd, rt.compute_units)
            rt.ops.attn_decode(qkv, qkv.shape[1], out, step.positions, step.token_seq, table, view.k, view.v,
                               view.page_size, nh, nkv, hd, self.scale, self.window, n_splits)
        elif aligned and rt.ops.attn_prefill_mfma_supported(rt.dtype, hd, view.page_size):
            queries = rt.prefill_queries or rt.ops.attn_prefill_queries(step.n_seqs, step.max_new, nh, nkv, hd, rt.compute_units)
            if queries == 32 and (hd % 32 or hd > 128):
                queries = 16
            rt.ops.attn_prefill_mfma(qkv, qkv.shape[1], out, step.positions, step.cu_seqlens, table, view.k, view.v,
                                     view.page_size, step.n_seqs, step.max_new, nh, nkv, hd, self.scale, self.window,
                                     queries=queries)
        else:
            # the generic kernel has one wavefront per (token, head); with few tokens over long key
            # ranges the ranges are cut so that the whole chip has work
            n_splits = 1
            if step.max_new == 1:
                span = step.max_len_after if not self.window else min(step.max_len_after, self.window)
                n_splits = max(1, min((span + 255) // 256, (4 * DECODE_TARGET_PER_UNIT * rt.compute_units) // max(1, qkv.shape[0] * nh)))
            rt.ops.attn_paged(qkv, qkv.shape[1], out, step.positions, step.token_seq, table, view.k, view.v,
                              view.page_size, nh, nkv, hd, self.scale, self.window, n_splits)
        return out
