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


class RandomWeightSource:
    """Random tensors made on the device, tensor by tensor, without a folder: for measurements,
    where writing and reading back gigabytes would only cost time.  Same distributions as
    :func:`random_tensors`; the values come from the device's generator."""

    def __init__(self, needs, seed: int, device, dtype: torch.dtype = torch.bfloat16,
                 std: float = 0.02, norm_std: float = 0.1):
        self._needs = {n.name: (i, n) for i, n in enumerate(needs)}
        self._seed, self._device, self._dtype = int(seed), device, dtype
        self._std, self._norm_std = std, norm_std

    def get(self, name: str) -> torch.Tensor:
        i, need = self._needs[name]
        g = torch.Generator(device=self._device).manual_seed((self._seed * 1_000_003 + i) & 0x7FFFFFFFFFFFFFFF)
        s = self._norm_std if len(need.shape) == 1 else self._std
        t = torch.empty(need.shape, dtype=torch.float32 if len(need.shape) == 1 else self._dtype, device=self._device)
        t.normal_(0.0, s, generator=g)
        return t
