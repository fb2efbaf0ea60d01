"""Random-weights mode: write a model folder from a configuration and a seed.

The reference has no such mode; it exists so that the loader, the engine and the plain
implementation of the tests can all read the very same tensors from disk.  Matrices and the
embedding are drawn from N(0, 0.02), norm weights from N(0, 0.1) (they act as 1 + w), one
tensor after the other in the order in which the model's parts list them, each from its own
generator seeded by (seed, position in that order), so a tensor's values do not depend on
the tensors before it.
"""
from __future__ import annotations

import json
import os
from typing import Dict, Optional

import torch

from ..config import find_architecture
from .safetensors_io import write_safetensors


def random_tensors(needs, seed: int, dtype: torch.dtype = torch.bfloat16,
                   std: float = 0.02, norm_std: float = 0.1) -> Dict[str, torch.Tensor]:
    out: Dict[str, torch.Tensor] = {}
    for i, need in enumerate(needs):
        g = torch.Generator().manual_seed((int(seed) * 1_000_003 + i) & 0x7FFFFFFFFFFFFFFF)
        s = norm_std if len(need.shape) == 1 else std
        out[need.name] = (torch.randn(need.shape, generator=g, dtype=torch.float32) * s).to(dtype)
    return out


def write_random_model(raw_config: dict, seed: int, out_dir: str,
                       dtype: torch.dtype = torch.bfloat16) -> str:
    """Write ``config.json`` and ``model.safetensors`` for ``raw_config`` into ``out_dir``."""
    from ..engine.model import tensor_needs          # parts state their tensors
    arch = find_architecture(raw_config)
    cfg = arch.parse(raw_config)
    spec = arch.spec(cfg, None)
    os.makedirs(out_dir, exist_ok=True)
    tensors = random_tensors(tensor_needs(spec), seed, dtype)
    write_safetensors(os.path.join(out_dir, "model.safetensors"), tensors)
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(raw_config, f, indent=1)
    return out_dir
