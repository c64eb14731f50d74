"""One step's batch: the tokens of several sequences packed into one run, with everything the
kernels need to know about where each token belongs."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Sequence

import torch


@dataclass
class Step:
    n_tokens: int
    n_seqs: int
    n_wanted: int
    token_ids: torch.Tensor      # int32 [tokens]
    positions: torch.Tensor      # int32 [tokens]  absolute position of each token in its sequence
    token_seq: torch.Tensor      # int32 [tokens]  index of the token's sequence in this step (-1: padding)
    seq_slots: torch.Tensor      # int32 [seqs]    cache slot of each sequence (-1: padding)
    cu_seqlens: torch.Tensor     # int32 [seqs+1]  first token of each sequence in the packed run
    lens_after: torch.Tensor     # int32 [seqs]    length of each sequence once this step has run
    want_rows: torch.Tensor      # int32 [wanted]  packed rows whose logits are asked for
    block_tables: Dict[int, torch.Tensor] = field(default_factory=dict)  # group -> int32 [seqs, width]
    max_new: int = 1             # most tokens any sequence brings
    max_position: int = 0        # largest position in the step
    max_len_after: int = 0
    is_decode: bool = False      # every sequence brings exactly one token
    host_slots: List[int] = field(default_factory=list)
    host_new: List[int] = field(default_factory=list)
    host_image: object = None    # the pinned host buffer the index arrays were copied from
    # (rows int32 [tokens], cell int64 [1]) or None.  Where rows[t] >= 0, token t is not token_ids[t] but
    # element rows[t] of the int32 array on the device whose address stands in the cell: a token that a
    # sampler left on the GPU and the host has not read.  Only given to an embedding that has forward_from.
    token_source: object = None


def build_step(entries, cache, device) -> Step:
    """entries: (slot, tokens, want) per sequence, or the same packed (cache.core.Packed).  The native
    core writes all index arrays into one host buffer, which goes to the device in one copy."""
    from ..cache.core import Packed
    packed = entries if isinstance(entries, Packed) else Packed(entries)
    news = packed.count_list()
    lengths = list(cache.lengths_of(packed))[:packed.n]
    T, B, R = sum(news), packed.n, packed.n_wanted
    max_after = max(past + n for past, n in zip(lengths, news))
    width = max(1, (max_after + cache.page_size - 1) // cache.page_size)
    size = cache.step_size(T, B, R, width)
    host = torch.empty(size, dtype=torch.int32, pin_memory=device.type == "cuda")
    cache.fill_step(packed, 0, 0, width, host.data_ptr(), size)
    dev = host.to(device, non_blocking=True)
    o = 0

    def take(n):
        nonlocal o
        v = dev[o:o + n]
        o += n
        return v

    token_ids, positions, token_seq = take(T), take(T), take(T)
    seq_slots, cu_seqlens, lens_after, want_rows = take(B), take(B + 1), take(B), take(R)
    block_tables = {gi: take(B * width).view(B, width) for gi in range(len(cache.groups))}
    step = Step(n_tokens=T, n_seqs=B, n_wanted=R, token_ids=token_ids, positions=positions, token_seq=token_seq,
                seq_slots=seq_slots, cu_seqlens=cu_seqlens, lens_after=lens_after, want_rows=want_rows,
                block_tables=block_tables, max_new=max(news), max_position=max_after - 1, max_len_after=max_after,
                is_decode=all(n == 1 for n in news), host_slots=packed.slot_list(), host_new=news)
    step.host_image = host   # the pinned source of the copy stays alive as long as the step
    return step
