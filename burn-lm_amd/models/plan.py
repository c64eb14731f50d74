"""The plan of a model: which parts make each layer, and in which order layers run.

The order is data: a list of places, each naming a layer.  A layer may be named by several
places (it then runs more than once with the same weights, each place keeping a cache of its
own), and a place may read the keys and values that an earlier place keeps instead of keeping
its own.  An architecture turns its configuration into such a plan; the model builder knows
nothing else about the architecture."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

from ..parts.base import PartSpec


class LayerPlan:
    """One layer: the kind of arrangement (a registered block, e.g. "pre_norm") and the part chosen
    for each role that this arrangement has.  Which roles there are is the block's business: the
    pre-norm block has ``mixer``, ``feed_forward``, ``mixer_norm`` and ``ffn_norm``; another block
    may have four norms, or no feed-forward.  Roles are given as a mapping or by keyword.
    ``position`` is a key into ModelPlan.positions; that encoding is handed to the layer's mixers."""

    def __init__(self, block: str, parts: Optional[Dict[str, PartSpec]] = None, position: Optional[str] = None,
                 **roles: PartSpec):
        self.block = block
        self.parts: Dict[str, PartSpec] = dict(parts or {})
        self.parts.update(roles)
        self.position = position
        for role, spec in self.parts.items():
            if not isinstance(spec, PartSpec):
                raise TypeError(f"layer plan: role {role!r} needs a PartSpec, got {type(spec).__name__}")

    def __getattr__(self, role):        # plan.mixer, plan.feed_forward, ...
        try:
            return self.__dict__["parts"][role]
        except KeyError:
            raise AttributeError(role) from None

    def __repr__(self):
        return f"LayerPlan({self.block!r}, {self.parts!r}, position={self.position!r})"


@dataclass(frozen=True)
class Place:
    layer: int
    reads_cache_of: Optional[int] = None  # index of an earlier place in the order


@dataclass
class ModelPlan:
    vocab_size: int
    width: int
    max_positions: int
    embedding: PartSpec
    layers: List[LayerPlan]
    order: List[Place]
    final_norm: PartSpec
    head: PartSpec
    positions: Dict[str, PartSpec] = field(default_factory=dict)
    stop_ids: Tuple[int, ...] = ()
    ignorable_tensors: Tuple[str, ...] = ()  # regular expressions of checkpoint names to skip silently
