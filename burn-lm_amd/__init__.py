"""burn-lm_amd: a small MI355X-native model library with generation.

From a model folder (config.json + safetensors, or seeded random weights) to generated tokens on
one GPU: typed configuration, a registry from architecture name to model, parts (mixer,
feed-forward, norm, position encoding, block) chosen layer by layer, a paged cache with a slot
per sequence, one step function, a generation loop, sampling, and hand-written HIP kernels for
gfx950.  The package directory is ``burn-lm_amd/``; it is imported as ``burn_lm_amd``.
"""
from . import registry  # noqa: F401
from . import parts as _parts  # noqa: F401  registers the part kinds
from . import models as _models  # noqa: F401  registers the architectures

__version__ = "0.1.0"


def load(folder, dtype="bfloat16", max_tokens=8192, **kw):
    """Engine for the model in ``folder`` (see ``engine.loading.load_engine``)."""
    from .engine.loading import load_engine
    return load_engine(folder, dtype=dtype, max_tokens=max_tokens, **kw)


def write_random_model(folder, config, seed=0, **kw):
    """Random-weights mode: write config.json and model.safetensors into ``folder``."""
    from .weights.random_init import write_model_folder
    return write_model_folder(folder, config, seed=seed, **kw)
