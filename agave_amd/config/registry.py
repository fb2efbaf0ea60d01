"""One registry from an architecture's name to its configuration and model spec.

Reference: ``Arch.detect`` maps the model-type string to an enum through an alias
table (``src/arch.zig:18-51``) and ``ModelStorage.initFromArch`` switches on it
(``src/models/model.zig:503-532``); an unknown name ends with "unsupported
architecture" (``src/main.zig:1010-1014``).  Here one table row holds the typed
configuration class; the class turns itself into a :class:`ModelSpec`, from which
the engine builds the model out of registered parts.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Callable, Dict, Iterable, Optional, Tuple

from .errors import ConfigError, UnsupportedArchitecture
from .spec import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str                                   # config.json "architectures"[0]
    model_types: Tuple[str, ...]                # accepted "model_type" values
    parse: Callable[[dict], object]             # raw config dict -> typed configuration
    # typed configuration, names of the checkpoint's tensors -> ModelSpec
    spec: Callable[[object, Optional[Iterable[str]]], ModelSpec]


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(arch: Architecture) -> None:
    _ARCHITECTURES[arch.name] = arch


def architectures() -> Tuple[str, ...]:
    return tuple(sorted(_ARCHITECTURES))


def find_architecture(raw: dict) -> Architecture:
    """Pick the row by ``architectures[0]``, else by ``model_type`` (also inside
    ``text_config``)."""
    names = raw.get("architectures") or []
    for n in names:
        if n in _ARCHITECTURES:
            return _ARCHITECTURES[n]
    types = [raw.get("model_type")]
    if isinstance(raw.get("text_config"), dict):
        types.append(raw["text_config"].get("model_type"))
    for arch in _ARCHITECTURES.values():
        if any(t in arch.model_types for t in types if t):
            return arch
    shown = names[0] if names else raw.get("model_type")
    raise UnsupportedArchitecture(
        f"unsupported architecture {shown!r}; supported: {', '.join(architectures())}")


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{path}: not found")
    with open(path, "r", encoding="utf-8") as f:
        try:
            raw = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return raw


def load_config(model_dir: str):
    """(architecture row, typed configuration) of a model folder."""
    raw = read_config_json(model_dir)
    arch = find_architecture(raw)
    return arch, arch.parse(raw)
