"""agave_amd: a small generation library for one GPU (MI355X, gfx950).

From a model folder (config.json + safetensors, or seeded random weights) through a typed
configuration and a registry to a model assembled from parts, a paged cache with a slot per
sequence, one step function over ragged batches, a generation loop with sampling, a command
line and a trace replay tool.  The compute path is hand-written HIP; there is no CPU path.
"""
from .config import ConfigError, Gemma3Config, UnsupportedArchitecture, load_config, register_architecture
from .weights import SafetensorsError, WeightError, write_random_model

__version__ = "0.1.0"


def __getattr__(name):
    # the engine imports the GPU machinery; keep `import agave_amd` light
    if name == "Engine":
        from .engine import Engine
        return Engine
    if name in ("SamplingParams", "GenerationResult"):
        from . import sampling
        return getattr(sampling, name)
    raise AttributeError(name)


__all__ = ["ConfigError", "UnsupportedArchitecture", "Gemma3Config", "load_config", "register_architecture",
           "SafetensorsError", "WeightError", "write_random_model", "Engine", "SamplingParams",
           "GenerationResult"]
