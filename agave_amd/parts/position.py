"""Position encodings applied to queries and keys.

``rope``: rotation of the pairs (i, i + rotary_dim/2) by ``pos/factor * theta^(-2i/rotary_dim)``
(``src/backend/kernels/cpu/rope.zig:11-48``; linear scaling multiplies the position by
``1/factor`` first, ``src/models/gemma3.zig:884-902``).  The frequencies are a table of 32-bit
floats, rounded once from their exact values; the angle and its sine and cosine are computed
in 32-bit inside the q/k kernel.  ``none``: nothing is applied.
"""
from __future__ import annotations

from typing import Optional, Tuple

import numpy as np
import torch

from ..config.spec import PositionSpec
from .base import BuildEnv, register


class RotaryPosition:
    def __init__(self, spec: PositionSpec, env: BuildEnv):
        if spec.rotary_dim < 2 or spec.rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even and >= 2, got {spec.rotary_dim}")
        if spec.theta <= 0 or spec.factor <= 0:
            raise ValueError("rope needs theta > 0 and factor > 0")
        i = np.arange(spec.rotary_dim // 2, dtype=np.float64)
        inv = np.exp(-np.log(float(spec.theta)) * (2.0 * i) / spec.rotary_dim)
        self.inv_freq = torch.from_numpy(inv.astype(np.float32)).to(env.device)
        self.pos_scale = float(np.float32(1.0) / np.float32(spec.factor))
        self.rotary_dim = spec.rotary_dim

    def fused_rotation(self) -> Tuple[Optional[torch.Tensor], float]:
        return self.inv_freq, self.pos_scale


class NoPosition:
    def __init__(self, spec: PositionSpec, env: BuildEnv):
        pass

    def fused_rotation(self) -> Tuple[Optional[torch.Tensor], float]:
        return None, 1.0


register("position", "rope", RotaryPosition)
register("position", "none", NoPosition)
