"""Parts a model is assembled from, and their registration under kind names."""
from .. import registry
from .attention import Attention
from .base import (Block, FeedForward, KVNeed, Mixer, Norm, Part, PartSpec, PositionEncoding, StateNeed,
                   TensorSpec)
from .block import PreNormBlock
from .embedding import Embedding, LMHead
from .norm_rms import RMSNorm
from .rope import RotaryEncoding
from .swiglu import SwiGLU

registry.register_part("mixer", "attention", Attention)
registry.register_part("feed_forward", "swiglu", SwiGLU)
registry.register_part("norm", "rmsnorm", RMSNorm)
registry.register_part("position", "rope", RotaryEncoding)
registry.register_part("block", "pre_norm", PreNormBlock)
registry.register_part("embedding", "table", Embedding)
registry.register_part("head", "linear", LMHead)
