"""Dense gated feed-forward: ``W_down (act(W_gate x) * (W_up x))``.

Reference: ``src/models/gemma3.zig:830-880`` (gate and up products, ``geluMul``, down
product); the activation is the tanh form of GELU
(``src/backend/kernels/cpu/activation.zig:69-113``).  Gate and up are one stacked product.

The activation is the spec's (``GatedFfnSpec.activation``, one of
``agave_amd.ops.kernels.GATE_ACTIVATIONS``).  With the tanh form of GELU and weights on the matrix
cores the product ends in the activation itself; with any other the stacked product is followed
by the elementwise kernel, which takes the activation as a parameter.
"""
from __future__ import annotations

from typing import List

import torch

from ..config.spec import GatedFfnSpec
from ..ops import kernels
from ..weights.loader import TensorNeed
from .base import BuildEnv, register
from .linear import Linear

FUSED_ACTIVATION = "gelu_tanh"          # the one that the matrix-core products end in


class GatedFfn:
    prompt_steps_can_be_recorded = True        # a multi-token step is the same launches whatever its tokens are
    takes_rows_to_be_normed = True             # its first product may make the normalised rows itself (NormedRows)

    def __init__(self, spec: GatedFfnSpec, weights, env: BuildEnv):
        if spec.activation not in kernels.GATE_ACTIVATIONS:
            raise ValueError(f"gated feed-forward: unsupported activation {spec.activation!r}; "
                             f"known: {sorted(kernels.GATE_ACTIVATIONS)}")
        self.spec = spec
        self.env = env
        # [gate; up] stacked; on the matrix cores their rows are interleaved so that the product ends in
        # GeGLU (the tanh form only: another activation takes the plain stack and the elementwise kernel)
        # (nor with a bias on gate or up: the fused product has no place for one)
        def bias(name):
            return weights.get(name) if name else None

        fused = spec.activation == FUSED_ACTIVATION and not (spec.gate_bias or spec.up_bias)
        self.gate_up = Linear([weights.get(spec.gate_proj), weights.get(spec.up_proj)], env, "gate_up",
                              interleave_ff=spec.intermediate if fused else 0,
                              biases=[bias(spec.gate_bias), bias(spec.up_bias)])
        self.down = Linear([weights.get(spec.down_proj)], env, "ffn_down", biases=[bias(spec.down_bias)])

    @staticmethod
    def tensor_needs(spec: GatedFfnSpec) -> List[TensorNeed]:
        needs = [TensorNeed(spec.gate_proj, (spec.intermediate, spec.hidden)),
                 TensorNeed(spec.up_proj, (spec.intermediate, spec.hidden)),
                 TensorNeed(spec.down_proj, (spec.hidden, spec.intermediate))]
        for name, size in ((spec.gate_bias, spec.intermediate), (spec.up_bias, spec.intermediate),
                           (spec.down_bias, spec.hidden)):
            if name:
                needs.append(TensorNeed(name, (size,)))
        return needs

    def forward(self, x: torch.Tensor, step) -> torch.Tensor:
        ff = self.spec.intermediate
        n = x.shape[0]
        act = self.env.workspace.get("ffn_act", n, ff, x.dtype)
        if not self.gate_up.forward_geglu(x, act):
            gu = self.gate_up.forward(x, tag="gate_up")
            kernels.gated_act(gu[:, :ff], gu[:, ff:], act, self.spec.activation)
        return self.down.forward(act, tag="ffn_down", slices_ok=True)    # the block adds it to the residual stream


register("ffn", "gated_dense", GatedFfn)
