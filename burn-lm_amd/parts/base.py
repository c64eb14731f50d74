"""What every part of a model is to the framework.

A model is put together from parts chosen by name: a *mixer* (attention, or anything else that
moves information between the tokens of a sequence), a *feed-forward*, a *norm*, a *position
encoding*, and a *block* that arranges them.  A part gets its sizes and constants as
parameters, names the checkpoint tensors it wants, and never learns which model it is in.

Interfaces (all tensors live on the GPU; ``x`` is ``[tokens, width]`` in the activation dtype,
``h`` the float32 residual stream of the same shape):

* ``Part.tensor_specs() -> {checkpoint name: TensorSpec}`` and ``Part.bind(tensors, rt)``.
* ``Norm.add_norm(h, delta, rows=None, write_h=True) -> x``: ``h += delta`` (if given), then
  the normalised rows (all rows, or the rows listed in ``rows``).  ``delta`` is ``[tokens, width]``
  in the activation dtype, or float32 ``[planes, tokens, width]`` whose planes are summed (a
  mixer or feed-forward may hand on the partial products of its last matrix product).
* ``Mixer.cache_need() -> KVNeed | StateNeed | None`` and
  ``Mixer.forward(x, step, view) -> delta``; ``view`` is what the cache holds for this place
  in the layer order (``KVView``, ``StateView`` or ``None``).
* ``FeedForward.forward(x, step) -> delta``.
* ``PositionEncoding.prepare(n_positions, rt)``, ``for_projection(w_q, w_k, heads, kv_heads)`` (the
  encoding may re-order the projections' rows when they are bound) and, for encodings that act on queries and keys,
  ``encode_and_store(qkv, step, view, heads, kv_heads, head_dim, store)``; the attention mixer calls
  ``project_encode_store(x, w_qkv, step, view, heads, kv_heads, head_dim)``, whose default is the
  projection followed by ``encode_and_store`` and which an encoding may fuse.
* ``Block.roles`` (role -> family of the parts it arranges), ``Block.cache_need()`` and
  ``Block.forward(h, delta, step, view) -> delta``: runs its parts; the returned delta has not
  been added to ``h`` yet (the next norm adds it, in float32).  A block with several parts that
  each keep something (an attention beside a mixer with a state) returns a tuple of needs and
  gets a tuple of views in the same order.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Tuple

import torch


@dataclass(frozen=True)
class TensorSpec:
    shape: Tuple[int, ...]
    kind: str = "float"  # "float": kept in bfloat16 / float32; "int": kept as int32


@dataclass(frozen=True)
class PartSpec:
    """Choice of a part: its registered kind, its parameters, and the checkpoint tensor name of
    each of its roles."""
    kind: str
    params: dict = field(default_factory=dict)
    names: Dict[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class KVNeed:
    """Keys and values per token.  window = 0 keeps every key; window = w keeps the last w.  Values
    may have a head size of their own (value_dim; 0: that of the keys) and a head count of their own
    (n_value_heads; 0: that of the keys); the attention of this library asks for equal ones."""
    n_kv_heads: int
    head_dim: int
    window: int = 0
    value_dim: int = 0
    n_value_heads: int = 0

    @property
    def v_dim(self):
        return self.value_dim or self.head_dim

    @property
    def v_heads(self):
        return self.n_value_heads or self.n_kv_heads


@dataclass(frozen=True)
class StateNeed:
    """State of fixed size per sequence, zeroed when a sequence starts."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class Part:
    # True if forward() only launches work on the current stream from device-side data, so that a
    # decode step through this part can be captured into a HIP graph and replayed.  A part that
    # reads the step's host-side lists (or syncs with the host) must leave this False.
    graph_safe = False

    def __init__(self, params: dict, names: Dict[str, str]):
        self.params = dict(params)
        self.names = dict(names)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {}

    def bind(self, tensors: Dict[str, torch.Tensor], rt) -> None:
        self.rt = rt

    # What a step costs at the least, for measurements against the machine's limits (a bound part answers):
    def step_bytes(self, rows: int) -> int:
        """Bytes of this part's tensors that a step over `rows` tokens has to read, each once."""
        return 0

    def step_flops(self, rows: int) -> int:
        """Floating-point operations of this part's matrix products for `rows` tokens."""
        return 0


class Norm(Part):
    def add_norm(self, h, delta, rows=None, write_h=True):
        raise NotImplementedError

    def rms_constants(self):
        """(gamma, eps) if this norm is ``v / sqrt(mean(v^2) + eps) * gamma`` of ``v = h + delta`` and
        nothing else, so that a part behind it may form it inside a kernel of its own; else None."""
        return None


class Mixer(Part):
    def cache_need(self):
        return None

    def mixing_flops(self, past: int, new: int) -> int:
        """Operations that move information between tokens (not the projections) when a sequence that
        holds `past` tokens gets `new` more."""
        return 0

    def forward(self, x, step, view):
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, x, step):
        raise NotImplementedError

    def forward_after_norm(self, h, delta, norm, step):
        """``forward(norm.add_norm(h, delta), step)``: the pending delta added to the residual stream,
        the norm, and this feed-forward.  A feed-forward may run the three as one kernel where it
        has one (it then must leave h as add_norm would)."""
        return self.forward(norm.add_norm(h, delta), step)


class PositionEncoding(Part):
    def prepare(self, n_positions: int, rt) -> None:
        pass

    def for_projection(self, w_q, w_k, heads: int, kv_heads: int):
        """Called by a mixer when it binds its query and key projections ([heads * head_dim, width]
        rows): returns (w_q, w_k, encoding) to use from then on.  An encoding may hand back
        re-ordered rows and a variant of itself that computes the same function on them."""
        return w_q, w_k, self

    def project_encode_store(self, x, w_qkv, step, view, heads, kv_heads, head_dim):
        """x @ w_qkv^T, then encode q and k by position and store k, v (unless view.store is
        False).  Returns the [tokens, (heads + 2 kv_heads) * head_dim] buffer whose first
        heads * head_dim columns are the encoded queries.  A subclass may fuse the steps."""
        qkv = self.rt.linear(x, w_qkv)
        self.encode_and_store(qkv, step, view, heads, kv_heads, head_dim, store=view.store)
        return qkv


class Block:
    """Arrangement of a layer's parts.  ``roles`` says which roles the arrangement has and of which
    family each is (the registry's families: mixer, feed_forward, norm); the model builder makes the
    part a layer plan names for every role and hands the block the mapping role -> part.  The parts
    are also reachable as attributes (``self.mixer`` ...).  A block whose cache need is not simply
    that of a role called ``mixer`` overrides ``cache_need``; it may return a tuple of needs, one for
    each of its parts that keeps something, and ``forward`` then gets a tuple of views in that order."""
    roles: Dict[str, str] = {}

    def __init__(self, parts: Dict[str, Part]):
        missing = [r for r in self.roles if r not in parts]
        unknown = [r for r in parts if r not in self.roles]
        if missing or unknown:
            raise ValueError(f"{type(self).__name__} has the roles {sorted(self.roles)}; the layer plan "
                             f"lacks {missing} and names unknown {unknown}")
        self._parts = dict(parts)
        for role, part in parts.items():
            setattr(self, role, part)

    def parts(self):
        """In the order the roles are declared (the order in which they are bound)."""
        return tuple(self._parts[r] for r in self.roles)

    def cache_need(self):
        mixer = self._parts.get("mixer")
        return mixer.cache_need() if mixer is not None else None

    def forward(self, h, delta, step, view):
        raise NotImplementedError
