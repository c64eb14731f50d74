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


@dataclass(frozen=True)
class LayerPlan:
    block: str            # kind of arrangement, e.g. "pre_norm"
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    ffn_norm: PartSpec
    position: Optional[str] = None  # key into ModelPlan.positions, handed to the mixer


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
