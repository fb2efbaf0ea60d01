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

# (branch, the norm after its sublayer | None[, base]).  ``base``: the tensor that holds the residual
# stream at this moment if that is not ``h`` (a product that made its own normalised rows summed the
# stream up in other memory, see NormedRows); whoever adds the branch reads the rows there and
# writes them to ``h``.
Pending = Optional[Tuple]


def unpack_pending(pending: Pending):
    """(branch, post norm, base), each None where there is none."""
    if pending is None:
        return None, None, None
    if len(pending) == 2:
        return pending[0], pending[1], None
    return pending


def add_branch(h: torch.Tensor, pending: Pending) -> None:
    """h += post(branch) for a branch that is still to be added (post None: h += branch).  The
    branch may be 32-bit slices [slices, rows, hidden] that add up to it."""
    branch, post, base = unpack_pending(pending)
    if branch is None:
        if base is not None:
            h.copy_(base)
        return
    if post is None:
        kernels.residual_norm(h, branch, None, 0.0, None, None, 0.0, src=base)
    elif isinstance(post, RmsNorm):
        kernels.residual_norm(h, branch, post.gain, post.eps, None, None, 0.0, src=base)
    else:
        if base is not None:
            h.copy_(base)
        post.add_to(h, branch)


class NormedRows:
    """``norm(h + post(branch))`` as a promise: the rows that a sublayer is given, not yet computed.

    Whoever takes them either calls :meth:`rows` (the norm's kernel runs, ``h`` holds the sum, and
    the rows come back as a tensor), or, being a product that can make them in its own kernel,
    takes :meth:`rms_arguments` and reports with :meth:`made_by_consumer` where it left the sum
    (it cannot write ``h`` in place: its other workgroups still read it).  ``shape`` and ``dtype``
    are those of the rows to be."""

    def __init__(self, h: torch.Tensor, pending: Pending, norm, workspace, dtype: torch.dtype):
        self.h, self.pending, self.norm = h, pending, norm
        self.workspace = workspace
        self.shape, self.dtype = h.shape, dtype
        self.base: Optional[torch.Tensor] = None      # afterwards: where the stream is, if not in h
        self._rows: Optional[torch.Tensor] = None
        self.taken = False

    def rows(self) -> torch.Tensor:
        if self._rows is None:
            if self.taken:
                raise RuntimeError("these rows were made inside a product's kernel and exist nowhere else")
            x = self.workspace.get("normed", self.shape[0], self.shape[1], self.dtype)
            self.norm.add_and_norm(self.h, self.pending, x)
            self._rows, self.taken = x, True
        return self._rows

    def rms_arguments(self):
        """(h_in, h_out, branch, post_gain, post_eps, pre_gain, pre_eps) if nothing was computed yet and
        both norms are RMS norms (the one on the branch may be absent), else None."""
        if self.taken:
            return None
        branch, post, base = unpack_pending(self.pending)
        if not isinstance(self.norm, RmsNorm) or (post is not None and not isinstance(post, RmsNorm)):
            return None
        h_in = base if base is not None else self.h
        h_out = None
        if branch is not None:
            h_out = self.h if base is not None else self.workspace.get("residual_aside", self.shape[0], self.shape[1],
                                                                       torch.float32)
        return (h_in, h_out, branch, post.gain if (branch is not None and post is not None) else None,
                post.eps if (branch is not None and post is not None) else 0.0, self.norm.gain, self.norm.eps)

    def made_by_consumer(self, h_in: torch.Tensor, h_out: Optional[torch.Tensor]) -> None:
        self.taken = True
        now = h_out if h_out is not None else h_in
        self.base = None if now is self.h or now.data_ptr() == self.h.data_ptr() else now


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
        branch, post, base = unpack_pending(pending)
        if branch is not None and post is not None and not isinstance(post, RmsNorm):
            add_branch(h, (branch, post, base))     # another kind of norm after the sublayer: its own kernel
            branch = post = base = None
        if rows is not None and (branch is not None or base is not None):
            add_branch(h, (branch, post, base))     # the fused kernel gathers rows only without a branch
            branch = post = base = None
        if branch is None and out is None:
            add_branch(h, (None, None, base))
            return
        kernels.residual_norm(h, branch, post.gain if (branch is not None and post) else None,
                              post.eps if (branch is not None and post) else 0.0,
                              out, self.gain if out is not None else None, self.eps if out is not None else 0.0, rows,
                              src=base)


register("norm", "rmsnorm", RmsNorm)
