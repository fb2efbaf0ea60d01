"""RMSNorm as a part: a gain vector and an eps; the arithmetic is in the residual kernels.

Reference: ``y = x * (1/sqrt(mean(x^2) + eps)) * g`` (``src/backend/kernels/cpu/norm.zig:7-40``);
for HF checkpoints ``g = 1 + w``, folded into a 32-bit gain once at load as the reference's
``warmNormCache`` does (``src/models/gemma3.zig:908-954``).
"""
from __future__ import annotations

from typing import List

import torch

from ..config.spec import NormSpec
from ..weights.loader import TensorNeed
from .base import BuildEnv, register


class RmsNorm:
    def __init__(self, spec: NormSpec, weights, env: BuildEnv):
        w = weights.get(spec.weight).to(torch.float32)
        if spec.add_one:
            w = w + 1.0
        self.gain = w.contiguous().to(env.device)
        self.eps = float(spec.eps)
        self.size = spec.size

    @staticmethod
    def tensor_needs(spec: NormSpec) -> List[TensorNeed]:
        return [TensorNeed(spec.weight, (spec.size,))]


register("norm", "rmsnorm", RmsNorm)
