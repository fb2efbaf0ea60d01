"""Dense gated feed-forward: ``W_down (act(W_gate x) * (W_up x))``.

Reference: ``src/models/gemma3.zig:830-880`` (gate and up products, ``geluMul``, down
product); the activation is the tanh form of GELU
(``src/backend/kernels/cpu/activation.zig:69-113``).  Gate and up are one stacked product.
"""
from __future__ import annotations

from typing import List

import torch

from ..config.spec import GatedFfnSpec
from ..ops import kernels
from ..weights.loader import TensorNeed
from .base import BuildEnv, register
from .linear import Linear

_ACTIVATIONS = ("gelu_tanh",)


class GatedFfn:
    def __init__(self, spec: GatedFfnSpec, weights, env: BuildEnv):
        if spec.activation not in _ACTIVATIONS:
            raise ValueError(f"gated feed-forward: unsupported activation {spec.activation!r}; known: {_ACTIVATIONS}")
        self.spec = spec
        self.env = env
        self.gate_up = Linear([weights.get(spec.gate_proj), weights.get(spec.up_proj)], env, "gate_up")
        self.down = Linear([weights.get(spec.down_proj)], env, "ffn_down")
        self.gate_up_fused = None   # [gate; up] with interleaved rows, for the product that ends in GeGLU
        if self.gate_up.packed is not None:
            from ..ops import gemm_mfma
            self.gate_up_fused = gemm_mfma.pack_weight(self.gate_up.weight, interleave_ff=spec.intermediate)
            self.gate_up.packed = None

    @staticmethod
    def tensor_needs(spec: GatedFfnSpec) -> List[TensorNeed]:
        return [TensorNeed(spec.gate_proj, (spec.intermediate, spec.hidden)),
                TensorNeed(spec.up_proj, (spec.intermediate, spec.hidden)),
                TensorNeed(spec.down_proj, (spec.hidden, spec.intermediate))]

    def forward(self, x: torch.Tensor, step) -> torch.Tensor:
        ff = self.spec.intermediate
        n = x.shape[0]
        act = self.env.workspace.get("ffn_act", n, ff, x.dtype)
        if self.gate_up_fused is not None and n <= 64 and x.dtype == torch.bfloat16:
            from ..ops import gemm_mfma
            gemm_mfma.skinny(x, self.gate_up_fused, act, ff, epilogue=1)
        else:
            gu = self.gate_up.forward(x, tag="gate_up")
            kernels.geglu(gu[:, :ff], gu[:, ff:], act)
        return self.down.forward(act, tag="ffn_down")


register("ffn", "gated_dense", GatedFfn)
