"""Arrangements of a layer's parts around the 32-bit residual stream ``h``.

``sandwich`` (``src/models/gemma3.zig:341-348, 708-709, 823-826, 835-836, 872-878``):

    h += post_mixer_norm(mixer(pre_mixer_norm(h)));  h += post_ffn_norm(ffn(pre_ffn_norm(h)))

``prenorm`` is the same without the two post norms.  A block never adds its last branch
itself: it returns it as *pending* ``(branch, norm | None)``, and whoever runs next (the
next block's first norm, or the model's end) hands it to the norm that comes next
(``norm.add_and_norm``), which adds it and computes itself, in one kernel where the kinds of
norm allow it, so that the residual stream is read and written once per sublayer.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from ..config.spec import LayerSpec
from ..weights.loader import TensorNeed
from .base import BuildEnv, lookup, register
from .norm import NormedRows, Pending, add_branch, rows_as_they_are


NORMED_ROWS_AS_A_PROMISE = 1        # up to this many rows a sublayer may make its normalised input itself


def add_pending_and_norm(h: torch.Tensor, pending: Pending, norm, out: Optional[torch.Tensor],
                         rows: Optional[torch.Tensor] = None) -> None:
    """h += post(branch) for a pending branch, then out = norm(h) if asked: the norm that comes
    next does it (``norm`` None: the branch is added and the rows are handed on as they are)."""
    if norm is None:
        if out is not None:
            rows_as_they_are(h, pending, out, rows)
        else:
            add_branch(h, pending)
    else:
        norm.add_and_norm(h, pending, out, rows)


class SandwichBlock:
    post_norms = True

    def __init__(self, spec: LayerSpec, weights, env: BuildEnv):
        self.spec = spec
        self.env = env

        def norm(ns):
            return lookup("norm", ns.kind)(ns, weights, env) if ns is not None else None
        self.pre_mixer = norm(spec.pre_mixer_norm)
        self.post_mixer = norm(spec.post_mixer_norm) if self.post_norms else None
        self.pre_ffn = norm(spec.pre_ffn_norm)
        self.post_ffn = norm(spec.post_ffn_norm) if self.post_norms else None
        if self.pre_mixer is None or (spec.ffn is not None and self.pre_ffn is None):
            raise ValueError("a block needs a norm before its mixer and before its feed-forward")
        self.mixer = lookup("mixer", spec.mixer.kind)(spec.mixer, weights, env)
        self.ffn = lookup("ffn", spec.ffn.kind)(spec.ffn, weights, env) if spec.ffn is not None else None
        self.hidden = self.pre_mixer.size

    @classmethod
    def tensor_needs(cls, spec: LayerSpec) -> List[TensorNeed]:
        needs: List[TensorNeed] = []
        norms = [spec.pre_mixer_norm, spec.pre_ffn_norm]
        if cls.post_norms:
            norms += [spec.post_mixer_norm, spec.post_ffn_norm]
        for ns in norms:
            if ns is not None:
                needs += lookup("norm", ns.kind).tensor_needs(ns)
        needs += lookup("mixer", spec.mixer.kind).tensor_needs(spec.mixer)
        if spec.ffn is not None:
            needs += lookup("ffn", spec.ffn.kind).tensor_needs(spec.ffn)
        return needs

    def forward(self, h: torch.Tensor, pending: Pending, step, memory: int, writes: bool) -> Pending:
        n = h.shape[0]
        if n <= NORMED_ROWS_AS_A_PROMISE:
            return self._forward_few_rows(h, pending, step, memory, writes)
        x = self.env.workspace.get("normed", n, self.hidden, self.env.dtype)
        self.pre_mixer.add_and_norm(h, pending, x)
        a = self.mixer.forward(x, step, memory, writes)
        pending = (a, self.post_mixer)
        if self.ffn is None:
            return pending
        self.pre_ffn.add_and_norm(h, pending, x)
        f = self.ffn.forward(x, step)
        return (f, self.post_ffn)

    def _forward_few_rows(self, h: torch.Tensor, pending: Pending, step, memory: int, writes: bool) -> Pending:
        """One row (a decode step of one sequence): a sublayer that says so is handed the normalised
        row as a promise, so that its first product can make it in its own kernel (two kernels a
        layer less, of seven that each cost their start and their end)."""
        ws, dtype = self.env.workspace, self.env.dtype
        x = NormedRows(h, pending, self.pre_mixer, ws, dtype)
        a = self.mixer.forward(x if getattr(self.mixer, "takes_rows_to_be_normed", False) else x.rows(), step, memory, writes)
        if not x.taken:
            raise RuntimeError(f"{type(self.mixer).__name__} was handed rows to be normalised and never took them")
        pending = (a, self.post_mixer, x.base)
        if self.ffn is None:
            return pending
        x = NormedRows(h, pending, self.pre_ffn, ws, dtype)
        f = self.ffn.forward(x if getattr(self.ffn, "takes_rows_to_be_normed", False) else x.rows(), step)
        if not x.taken:
            raise RuntimeError(f"{type(self.ffn).__name__} was handed rows to be normalised and never took them")
        return (f, self.post_ffn, x.base)


class PreNormBlock(SandwichBlock):
    post_norms = False


register("block", "sandwich", SandwichBlock)
register("block", "prenorm", PreNormBlock)
