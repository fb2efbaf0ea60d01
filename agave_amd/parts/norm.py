"""Norms as parts.  A norm owns two things a block asks of it around the 32-bit residual stream
``h``: adding a branch it normalises (``h += norm(branch)``, the norm *after* a sublayer), and
normalising ``h`` for the next sublayer (the norm *before* it), optionally of chosen rows only.
A block never does either itself; it calls ``add_and_norm`` of the norm that comes next, which
also receives the branch that is still to be added (with the norm after its sublayer, if any),
so that a kind of norm that can do both in one pass over ``h`` does so.

:class:`Norm` is the general form: ``apply`` and ``add_to`` are what a new kind writes, and
``add_and_norm`` is put together from them.  :class:`RmsNorm` overrides it with the one fused
kernel when the norm after the sublayer is an RMS norm too (or none).

RMSNorm: ``y = x * (1/sqrt(mean(x^2) + eps)) * g`` (``src/backend/kernels/cpu/norm.zig:7-40``);
for HF checkpoints ``g = 1 + w``, folded into a 32-bit gain once at load as the reference's
``warmNormCache`` does (``src/models/gemma3.zig:908-954``).
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from ..config.spec import NormSpec
from ..ops import kernels
from ..weights.loader import TensorNeed
from .base import BuildEnv, register

Pending = Optional[Tuple[torch.Tensor, Optional[object]]]     # (branch, the norm after its sublayer | None)


def add_branch(h: torch.Tensor, pending: Pending) -> None:
    """h += post(branch) for a branch that is still to be added (post None: h += branch).  The
    branch may be 32-bit slices [slices, rows, hidden] that add up to it."""
    if pending is None:
        return
    branch, post = pending
    if post is None:
        kernels.residual_norm(h, branch, None, 0.0, None, None, 0.0)
    else:
        post.add_to(h, branch)


def rows_as_they_are(h: torch.Tensor, pending: Pending, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
    """What stands where a norm would for a model without one: the pending branch is added and
    the (chosen) rows of ``h`` are handed on, rounded to ``out``'s element type."""
    add_branch(h, pending)
    kernels.gather_rows(h, rows, out)


class Norm:
    """The interface of a norm, with ``add_and_norm`` composed of the two pieces a kind must
    write.  Fields: ``size`` (the length of the rows it normalises)."""
    size: int

    def apply(self, x: torch.Tensor, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
        """out[i] = norm(x[rows[i]]) (all rows if ``rows`` is None).  ``x`` is the 32-bit residual
        stream [n, size]; ``out`` has the activations' element type."""
        raise NotImplementedError

    def add_to(self, h: torch.Tensor, branch: torch.Tensor) -> None:
        """h += norm(branch).  ``branch`` is [n, size] in the activations' element type, or 32-bit
        slices [slices, n, size] that add up to it."""
        raise NotImplementedError

    def add_and_norm(self, h: torch.Tensor, pending: Pending, out: Optional[torch.Tensor],
                     rows: Optional[torch.Tensor] = None) -> None:
        """Add the pending branch to ``h``, then out = self(h) (of the chosen rows) if asked."""
        add_branch(h, pending)
        if out is not None:
            self.apply(h, out, rows)


class RmsNorm(Norm):
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

    def apply(self, x, out, rows=None) -> None:
        kernels.residual_norm(x, None, None, 0.0, out, self.gain, self.eps, rows)

    def add_to(self, h, branch) -> None:
        kernels.residual_norm(h, branch, self.gain, self.eps, None, None, 0.0)

    def add_and_norm(self, h, pending, out, rows=None) -> None:
        """One kernel adds the branch (through the RMS norm after its sublayer, if it has one) and
        computes this norm, reading and writing ``h`` once."""
        branch, post = pending if pending is not None else (None, None)
        if branch is not None and post is not None and not isinstance(post, RmsNorm):
            post.add_to(h, branch)              # another kind of norm after the sublayer: its own kernel
            branch = post = None
        if rows is not None and branch is not None:
            add_branch(h, (branch, post))       # the fused kernel gathers rows only without a branch
            branch = post = None
        if branch is None and out is None:
            return
        kernels.residual_norm(h, branch, post.gain if (branch is not None and post) else None,
                              post.eps if (branch is not None and post) else 0.0,
                              out, self.gain if out is not None else None, self.eps if out is not None else 0.0, rows)


register("norm", "rmsnorm", RmsNorm)
