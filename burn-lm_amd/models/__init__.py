"""Architectures: each module registers itself under the names its config.json uses."""
from . import llama  # noqa: F401
from .plan import LayerPlan, ModelPlan, Place  # noqa: F401
