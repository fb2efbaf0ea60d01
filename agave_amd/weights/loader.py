"""Resolving a model's tensors by name, with one error that lists everything wrong.

Reference: the reference looks tensors up lazily on every forward and fails at the first
missing one (``error.MissingTensor``, ``src/models/gemma3.zig:352, 450``).  Here every part
of the model states the tensors it needs (name and shape); all of them are checked before
anything is read, and a single :class:`WeightError` lists the missing names, the names the
checkpoint holds that no part asked for, and the shapes that do not fit.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Iterable, List, Sequence, Tuple

import torch

from .safetensors_io import Checkpoint


@dataclass(frozen=True)
class TensorNeed:
    name: str
    shape: Tuple[int, ...]


class WeightError(ValueError):
    def __init__(self, missing: Sequence[str], unexpected: Sequence[str],
                 wrong_shape: Sequence[Tuple[str, Tuple[int, ...], Tuple[int, ...]]], where: str = ""):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        lines = [f"weights of {where or 'the model'} do not fit its configuration:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + ", ".join(
                f"{n} is {list(got)}, needs {list(want)}" for n, got, want in self.wrong_shape))
        super().__init__("\n".join(lines))


def check_tensors(have: Dict[str, Tuple[int, ...]], needs: Iterable[TensorNeed], where: str = "") -> None:
    """Raise one :class:`WeightError` if ``have`` (name -> shape) and ``needs`` differ."""
    needs = list(needs)
    wanted = {n.name for n in needs}
    missing = [n.name for n in needs if n.name not in have]
    unexpected = sorted(n for n in have if n not in wanted)
    wrong = [(n.name, tuple(have[n.name]), tuple(n.shape)) for n in needs
             if n.name in have and tuple(have[n.name]) != tuple(n.shape)]
    if missing or unexpected or wrong:
        raise WeightError(missing, unexpected, wrong, where)


class WeightSource:
    """What the model builder reads tensors from: a checked checkpoint."""

    def __init__(self, checkpoint: Checkpoint, needs: Iterable[TensorNeed]):
        check_tensors({n: checkpoint.shape(n) for n in checkpoint.names()}, needs, checkpoint.model_dir)
        self._ckpt = checkpoint

    def get(self, name: str) -> torch.Tensor:
        """CPU tensor in its kept dtype (bfloat16, float32 or int32)."""
        return self._ckpt.read(name)


class DictWeightSource:
    """The same over tensors already in memory (tests, random weights without a folder)."""

    def __init__(self, tensors: Dict[str, torch.Tensor], needs: Iterable[TensorNeed], where: str = "dict"):
        check_tensors({n: tuple(t.shape) for n, t in tensors.items()}, needs, where)
        self._tensors = tensors

    def get(self, name: str) -> torch.Tensor:
        t = self._tensors[name]
        if t.dtype in (torch.bfloat16, torch.float32, torch.int32):
            return t
        return t.to(torch.float32 if t.is_floating_point() else torch.int32)
