"""Typed configurations and the architecture registry."""
from .errors import ConfigError, UnsupportedArchitecture
from .gemma3 import Gemma3Config
from .registry import (Architecture, architectures, find_architecture, load_config,
                       read_config_json, register_architecture)
from .spec import (AttentionSpec, FeedForwardSpec, GatedFfnSpec, LayerSpec, MixerSpec,
                   ModelSpec, NormSpec, PositionSpec, RunEntry)

register_architecture(Architecture(
    name=Gemma3Config.architecture,
    model_types=("gemma3_text", "gemma3"),          # aliases of src/arch.zig:22-24 that name this model
    parse=Gemma3Config.from_dict,
    spec=lambda cfg, names=None: cfg.model_spec(names)))

__all__ = [
    "ConfigError", "UnsupportedArchitecture", "Gemma3Config", "Architecture", "architectures",
    "find_architecture", "load_config", "read_config_json", "register_architecture",
    "AttentionSpec", "FeedForwardSpec", "GatedFfnSpec", "LayerSpec", "MixerSpec", "ModelSpec",
    "NormSpec", "PositionSpec", "RunEntry"]
