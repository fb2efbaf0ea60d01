"""Resolving a model's tensors by name, with one error that lists everything wrong.

Reference: the reference looks tensors up lazily on every forward and fails at the first
missing one (``error.MissingTensor``, ``src/models/gemma3.zig:352, 450``), and maps a stored
element type it does not know to ``.unknown`` (``src/format/safetensors.zig:1605-1616``: F32,
F16 and BF16 are the floating-point types it takes).  Here every part of the model states the
tensors it needs (name, shape, and whether it holds floats or integers); all of them are
checked before anything is read, and a single :class:`WeightError` lists the missing names, the
names the checkpoint holds that no part asked for, the shapes that do not fit and the tensors
stored in an element type that their use does not take.  The reference's lookup by name never
sees the tensors it does not ask for (``src/format/safetensors.zig:333-349``: the name, then the
name under each prefix of ``hf_prefixes``, ``:517-521``), so a folder that also holds a vision
tower loads there; here an architecture states which names are its own
(``ModelSpec.tensor_scope``): a name nobody asked for is an error inside that scope and is passed
over, and counted, outside it.
"""
from __future__ import annotations

import sys
from dataclasses import dataclass
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import torch

from .safetensors_io import Checkpoint


FLOAT_STORAGE = ("BF16", "F16", "F32")                       # what a matrix or vector of floats may be stored as
INT_STORAGE = ("I64", "I32", "I16", "I8", "U8")              # what an integer table may be stored as
_STORAGE_OF = {torch.bfloat16: "BF16", torch.float16: "F16", torch.float32: "F32", torch.float64: "F64",
               torch.int64: "I64", torch.int32: "I32", torch.int16: "I16", torch.int8: "I8", torch.uint8: "U8",
               torch.bool: "BOOL"}


@dataclass(frozen=True)
class TensorNeed:
    name: str
    shape: Tuple[int, ...]
    kind: str = "float"         # "float": a matrix or vector of floats; "int": an integer table

    def accepts(self, stored: str) -> bool:
        return stored in (FLOAT_STORAGE if self.kind == "float" else INT_STORAGE)


class WeightError(ValueError):
    def __init__(self, missing: Sequence[str], unexpected: Sequence[str],
                 wrong_shape: Sequence[Tuple[str, Tuple[int, ...], Tuple[int, ...]]], where: str = "",
                 wrong_dtype: Sequence[Tuple[str, str, str]] = ()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)            # (name, stored as, kind needed)
        lines = [f"weights of {where or 'the model'} do not fit its configuration:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + ", ".join(
                f"{n} is {list(got)}, needs {list(want)}" for n, got, want in self.wrong_shape))
        if self.wrong_dtype:
            lines.append(f"  wrong element type ({len(self.wrong_dtype)}): " + ", ".join(
                f"{n} is stored as {got}, needs one of {'/'.join(FLOAT_STORAGE if kind == 'float' else INT_STORAGE)}"
                for n, got, kind in self.wrong_dtype))
        super().__init__("\n".join(lines))


def check_tensors(have: Dict[str, Tuple[int, ...]], needs: Iterable[TensorNeed], where: str = "",
                  stored: Optional[Dict[str, str]] = None,
                  scope: Optional[Sequence[str]] = None) -> List[str]:
    """Raise one :class:`WeightError` if ``have`` (name -> shape) and ``needs`` differ, or if
    ``stored`` (name -> the container's name of the element type) holds a type that a tensor's
    use does not take.  ``scope`` lists the name prefixes that belong to the model: a name that
    no part asked for is an error if it starts with one of them (or if ``scope`` is None) and
    is returned, as one of the names passed over, if it does not."""
    needs = list(needs)
    wanted = {n.name for n in needs}
    missing = [n.name for n in needs if n.name not in have]
    unasked = sorted(n for n in have if n not in wanted)
    if scope is None:
        unexpected, passed_over = unasked, []
    else:
        own = tuple(scope)
        unexpected = [n for n in unasked if n.startswith(own)]
        passed_over = [n for n in unasked if not n.startswith(own)]
    wrong = [(n.name, tuple(have[n.name]), tuple(n.shape)) for n in needs
             if n.name in have and tuple(have[n.name]) != tuple(n.shape)]
    bad_type = []
    if stored is not None:
        bad_type = [(n.name, stored[n.name], n.kind) for n in needs
                    if n.name in stored and not n.accepts(stored[n.name])]
    if missing or unexpected or wrong or bad_type:
        raise WeightError(missing, unexpected, wrong, where, bad_type)
    return passed_over


def _report_passed_over(names: Sequence[str], where: str) -> None:
    if names:
        heads = sorted({".".join(n.split(".")[:2]) for n in names})
        shown = ", ".join(heads[:4]) + (", ..." if len(heads) > 4 else "")
        print(f"[agave_amd] {where}: {len(names)} tensors that are not the model's were passed over ({shown})",
              file=sys.stderr, flush=True)


class WeightSource:
    """What the model builder reads tensors from: a checked checkpoint."""

    def __init__(self, checkpoint: Checkpoint, needs: Iterable[TensorNeed],
                 scope: Optional[Sequence[str]] = None):
        self.passed_over = check_tensors(
            {n: checkpoint.shape(n) for n in checkpoint.names()}, needs, checkpoint.model_dir,
            stored={n: checkpoint.stored_dtype(n) for n in checkpoint.names()}, scope=scope)
        _report_passed_over(self.passed_over, checkpoint.model_dir)
        self._ckpt = checkpoint

    def get(self, name: str) -> torch.Tensor:
        """CPU tensor in its kept dtype (bfloat16, float16, float32 or int32)."""
        return self._ckpt.read(name)


class DictWeightSource:
    """The same over tensors already in memory (tests, random weights without a folder)."""

    def __init__(self, tensors: Dict[str, torch.Tensor], needs: Iterable[TensorNeed], where: str = "dict",
                 scope: Optional[Sequence[str]] = None):
        self.passed_over = check_tensors(
            {n: tuple(t.shape) for n, t in tensors.items()}, needs, where,
            stored={n: _STORAGE_OF.get(t.dtype, str(t.dtype)) for n, t in tensors.items()}, scope=scope)
        _report_passed_over(self.passed_over, where)
        self._tensors = tensors

    def get(self, name: str) -> torch.Tensor:
        t = self._tensors[name]
        if t.dtype in (torch.bfloat16, torch.float16, torch.float32, torch.int32):
            return t
        return narrow_to_int32(t, name)


def narrow_to_int32(t: torch.Tensor, name: str) -> torch.Tensor:
    """An integer table as int32; values that int32 cannot hold are an error, not a wrap-around."""
    if t.numel() and t.dtype in (torch.int64, torch.uint8, torch.int16, torch.int8):
        lo, hi = int(t.min()), int(t.max())
        if lo < -2 ** 31 or hi > 2 ** 31 - 1:
            raise ValueError(f"tensor {name!r}: values {lo}..{hi} do not fit the 32-bit integers tables are kept in")
    return t.to(torch.int32)
