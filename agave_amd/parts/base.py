"""What every part of a layer looks like to the model builder, and the part registries.

A part is built from its spec (sizes and constants as plain data) and a weight source; it
states the tensors it needs before anything is loaded; and it runs on the tokens of one
step.  No part knows which model it is in: the block arrangement asks the registries for
the kinds that the layer's spec names.

Interfaces (duck-typed; the classes below document them):

* norm:        ``tensor_needs(spec)``, ``__init__(spec, weights, env)``, field ``size``,
               ``apply(x, out, rows=None)`` (out = norm of the 32-bit rows x, or of the chosen ones),
               ``add_to(h, branch)`` (h += norm(branch)) and ``add_and_norm(h, pending, out, rows=None)``,
               which :class:`agave_amd.parts.norm.Norm` composes of the two; blocks and the model's end
               only ever call the last.
* position:    ``__init__(spec, env)``, ``fused_rotation() -> (inv_freq | None, pos_scale)`` when the
               q/k kernel can apply it (a rotation of pairs, or nothing), else ``apply(q, k, step)``:
               in place on the normalised rows q [N, heads*head_dim] and k [N, kv_heads*head_dim]
               (k is None in a run that appends nothing), positions in ``step.tok_pos``.
* mixer:       ``tensor_needs(spec)``, ``__init__(spec, weights, env)``, ``kv_need() -> GroupKey | None``,
               ``state_need() -> StateNeed | None``,
               ``forward(x[N, hidden], step, memory, writes) -> [N, hidden]`` (or slices of it, as below).
* feed-forward: ``tensor_needs(spec)``, ``__init__(spec, weights, env)``, ``forward(x[N, hidden], step) -> [N, hidden]``
               (or float32 [slices, N, hidden] whose slices add up to it: the block's residual kernel adds them).
* block:       ``tensor_needs(spec)``, ``__init__(spec, weights, env)``,
               ``forward(h, pending, step, memory, writes) -> pending`` (see ``block.py``).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional

import torch


@dataclass
class BuildEnv:
    """Where and in which element type the parts are built."""
    dtype: torch.dtype                 # torch.float32 or torch.bfloat16: activations and cache
    device: torch.device
    workspace: "Workspace"
    keep_stored_precision: bool = True   # a matrix stored in 32-bit stays so in a bfloat16 engine
    kept_32bit: List[str] = field(default_factory=list)    # names of the products that therefore miss the matrix cores

    def weight_dtype(self, stored: torch.dtype) -> torch.dtype:
        """The element type a matrix (or the embedding table) stored as ``stored`` is held in.  A
        32-bit engine widens everything (exactly).  A bfloat16 engine keeps bfloat16, casts half
        precision to bfloat16, and keeps 32-bit storage unless it was told to cast that too."""
        if stored not in (torch.float32, torch.bfloat16, torch.float16):
            raise TypeError(f"a weight matrix must hold floats (bfloat16, float16 or float32), got {stored}")
        if self.dtype == torch.float32:
            return torch.float32
        if stored == torch.float32 and self.keep_stored_precision:
            return torch.float32
        return self.dtype


class Workspace:
    """Named device buffers that are reused from step to step, so a step allocates nothing
    once its sizes have been seen.  ``generation`` changes whenever a buffer had to grow (the
    smaller one it replaces is freed), which tells a captured graph that its addresses are
    stale; a buffer under a new name moves nothing and leaves the graphs alone.  ``allocations``
    counts both: nothing may be allocated while a graph is being recorded."""

    def __init__(self, device: torch.device):
        self.device = device
        self._buffers: Dict[tuple, torch.Tensor] = {}
        self._views: Dict[tuple, torch.Tensor] = {}        # (name, cols, dtype, rows) -> the first rows of the buffer
        self.generation = 0
        self.allocations = 0

    def get(self, name: str, rows: int, cols: int, dtype: torch.dtype) -> torch.Tensor:
        # (a step asks for a few hundred buffers: the views are kept, one dictionary lookup each)
        vkey = (name, cols, dtype, rows)
        view = self._views.get(vkey)
        if view is not None:
            return view
        key = (name, cols, dtype)
        buf = self._buffers.get(key)
        if buf is None or buf.shape[0] < rows:
            cap = max(rows, 1)
            if buf is not None:
                cap = max(cap, buf.shape[0] * 2)
                self.generation += 1
                self._views.clear()                          # views of the buffer that gives way (and what was made of them)
            buf = torch.empty((cap, cols), dtype=dtype, device=self.device)
            self._buffers[key] = buf
            self.allocations += 1
        if len(self._views) > 4096:
            self._views.clear()
        view = self._views[vkey] = buf[:rows]
        return view

    def get3(self, name: str, slices: int, rows: int, cols: int, dtype: torch.dtype) -> torch.Tensor:
        """``slices`` buffers of [rows, cols] behind each other, as one [slices, rows, cols] tensor."""
        flat = self.get(name, slices * rows, cols, dtype)
        key = (name, cols, dtype, slices * rows, slices)
        view = self._views.get(key)
        if view is None or view.data_ptr() != flat.data_ptr():
            view = self._views[key] = flat.view(slices, rows, cols)
        return view

    def columns(self, t: torch.Tensor, bounds) -> tuple:
        """``t[:, bounds[i]:bounds[i + 1]]`` for every i, made once per tensor kept here and bounds."""
        key = ("columns", t.data_ptr(), t.shape[0], t.stride(0), bounds)
        got = self._views.get(key)
        if got is None:
            got = self._views[key] = tuple(t[:, lo:hi] for lo, hi in zip(bounds[:-1], bounds[1:]))
        return got

    def reserve(self, name: str, rows: int, cols: int, dtype: torch.dtype) -> None:
        self.get(name, rows, cols, dtype)

    def zeros(self, name: str, n: int, dtype: torch.dtype = torch.int32) -> torch.Tensor:
        """A zero-filled buffer that is zeroed only when it is made: for counters that every
        kernel using them leaves at zero again."""
        key = ("zeros:" + name, 0, dtype)
        buf = self._buffers.get(key)
        if buf is None or buf.numel() < n:
            if buf is not None:
                self.generation += 1
            buf = torch.zeros(max(n, 1024 if buf is None else 2 * buf.numel()), dtype=dtype, device=self.device)
            self._buffers[key] = buf
            self.allocations += 1
        return buf[:n]


_REGISTRIES: Dict[str, Dict[str, Callable]] = {"norm": {}, "position": {}, "mixer": {}, "ffn": {}, "block": {}}


def register(category: str, kind: str, cls: Callable) -> None:
    """Make ``cls`` the implementation of ``kind`` in ``category`` (norm, position, mixer, ffn,
    block).  A later registration of the same kind replaces the earlier one."""
    if category not in _REGISTRIES:
        raise KeyError(f"unknown part category {category!r}; known: {sorted(_REGISTRIES)}")
    _REGISTRIES[category][kind] = cls


def lookup(category: str, kind: str) -> Callable:
    try:
        return _REGISTRIES[category][kind]
    except KeyError:
        raise KeyError(f"no {category} part of kind {kind!r} is registered; known: "
                       f"{sorted(_REGISTRIES.get(category, {}))}") from None


def registered(category: str) -> List[str]:
    return sorted(_REGISTRIES[category])


def part_tensors(obj, _seen=None, _depth=0):
    """Every device tensor a part (and the parts inside it) holds, each once."""
    seen = _seen if _seen is not None else set()
    if isinstance(obj, torch.Tensor):
        if obj.data_ptr() not in seen:
            seen.add(obj.data_ptr())
            yield obj
        return
    if _depth > 6 or obj is None or isinstance(obj, (BuildEnv, Workspace, str, int, float, bool)):
        return
    if isinstance(obj, (list, tuple)):
        for x in obj:
            yield from part_tensors(x, seen, _depth + 1)
        return
    if isinstance(obj, dict):
        for x in obj.values():
            yield from part_tensors(x, seen, _depth + 1)
        return
    if hasattr(obj, "__dict__") and not hasattr(obj, "__dataclass_fields__"):
        for v in vars(obj).values():
            yield from part_tensors(v, seen, _depth + 1)
