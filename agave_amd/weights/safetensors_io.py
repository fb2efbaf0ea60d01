"""Reading and writing the safetensors container, by tensor name.

Reference: ``SafeTensorsDir.open`` (``src/format/safetensors.zig:97-279``) takes the shard
list from ``model.safetensors.index.json`` or scans the folder for ``*.safetensors``
(``:117-168, 1345-1384``), maps each shard, reads the 8-byte little-endian header length,
checks it against the file size and parses the JSON header
``{name: {dtype, shape, data_offsets}}``, skipping ``__metadata__`` (``:1633-1728``).
The same checks are made here; every failure is a :class:`SafetensorsError` that names the
file and what is wrong with it.

Tensors come back as CPU tensors over the mapped file (no copy): bfloat16 stays bfloat16, a
tensor stored in 32-bit floats stays so, half precision stays half precision until the part
that uses it casts it to the engine's element type, and integer tables become int32 (a value
that does not fit is an error).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
import warnings
from dataclasses import dataclass
from typing import Dict, Iterable, List, Mapping, Tuple

import torch


class SafetensorsError(ValueError):
    pass


# name in the header -> (torch dtype of the stored bytes, bytes per element)
_STORED = {
    "BF16": (torch.bfloat16, 2), "F32": (torch.float32, 4), "F16": (torch.float16, 2),
    "F64": (torch.float64, 8), "I64": (torch.int64, 8), "I32": (torch.int32, 4),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_WRITE_NAME = {torch.bfloat16: "BF16", torch.float32: "F32", torch.float16: "F16",
               torch.float64: "F64", torch.int64: "I64", torch.int32: "I32",
               torch.int16: "I16", torch.int8: "I8", torch.uint8: "U8", torch.bool: "BOOL"}


def kept_dtype(stored: str) -> torch.dtype:
    """The dtype a stored tensor is kept in after loading."""
    if stored == "BF16":
        return torch.bfloat16
    if stored == "F16":
        return torch.float16
    if stored in ("F32", "F64"):
        return torch.float32
    return torch.int32


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str
    shape: Tuple[int, ...]
    shard: int
    begin: int          # byte range inside the shard's data section
    end: int


class _Shard:
    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: file is {size} bytes, too short for a header length")
        self._file = open(path, "rb")
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ)
        (hlen,) = struct.unpack("<Q", self._map[:8])
        if hlen > size - 8:
            raise SafetensorsError(f"{path}: header length {hlen} exceeds the file ({size} bytes)")
        try:
            self.header = json.loads(self._map[8:8 + hlen].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON ({e})") from None
        if not isinstance(self.header, dict):
            raise SafetensorsError(f"{path}: header must be a JSON object")
        self.data_start = 8 + hlen
        self.data_size = size - self.data_start

    def view(self, begin: int, end: int) -> memoryview:
        return memoryview(self._map)[self.data_start + begin:self.data_start + end]


def _safe_shard_name(name: str) -> bool:
    # no path separators or parent references (src/format/safetensors.zig:1333-1340)
    return bool(name) and "/" not in name and "\\" not in name and ".." not in name and name.endswith(".safetensors")


class Checkpoint:
    """All tensors of a model folder, addressed by name."""

    def __init__(self, model_dir: str):
        self.model_dir = model_dir
        if not os.path.isdir(model_dir):
            raise SafetensorsError(f"{model_dir}: not a directory")
        shard_names = self._discover(model_dir)
        if not shard_names:
            raise SafetensorsError(f"{model_dir}: no .safetensors file found")
        self._shards: List[_Shard] = []
        self.entries: Dict[str, TensorEntry] = {}
        for si, sname in enumerate(shard_names):
            shard = _Shard(os.path.join(model_dir, sname))
            self._shards.append(shard)
            for name, meta in shard.header.items():
                if name == "__metadata__":
                    continue
                self.entries[name] = self._entry(shard, si, name, meta)

    @staticmethod
    def _discover(model_dir: str) -> List[str]:
        index = os.path.join(model_dir, "model.safetensors.index.json")
        if os.path.isfile(index):
            with open(index, "r", encoding="utf-8") as f:
                try:
                    wm = json.load(f).get("weight_map", {})
                except json.JSONDecodeError as e:
                    raise SafetensorsError(f"{index}: not valid JSON ({e})") from None
            names: List[str] = []
            for shard in wm.values():
                if not _safe_shard_name(shard):
                    raise SafetensorsError(f"{index}: bad shard name {shard!r}")
                if shard not in names:
                    names.append(shard)
            missing = [n for n in names if not os.path.isfile(os.path.join(model_dir, n))]
            if missing:
                raise SafetensorsError(f"{index}: shard files not found: {', '.join(missing)}")
            if names:
                return names
        return sorted(n for n in os.listdir(model_dir) if n.endswith(".safetensors"))

    @staticmethod
    def _entry(shard: _Shard, si: int, name: str, meta) -> TensorEntry:
        where = f"{shard.path}: tensor {name!r}"
        if not isinstance(meta, dict) or not all(k in meta for k in ("dtype", "shape", "data_offsets")):
            raise SafetensorsError(f"{where}: entry needs dtype, shape and data_offsets")
        dtype = meta["dtype"]
        if dtype not in _STORED:
            raise SafetensorsError(f"{where}: unsupported dtype {dtype!r}")
        shape = tuple(int(d) for d in meta["shape"])
        if any(d < 0 for d in shape):
            raise SafetensorsError(f"{where}: negative dimension in shape {list(shape)}")
        try:
            begin, end = (int(x) for x in meta["data_offsets"])
        except (TypeError, ValueError):
            raise SafetensorsError(f"{where}: data_offsets must be two integers") from None
        if begin < 0 or end < begin:
            raise SafetensorsError(f"{where}: data_offsets end {end} before start {begin}")
        if end > shard.data_size:
            raise SafetensorsError(f"{where}: data range [{begin}, {end}) runs past the file's "
                                   f"data section ({shard.data_size} bytes)")
        count = 1
        for d in shape:
            count *= d
        if count * _STORED[dtype][1] != end - begin:
            raise SafetensorsError(f"{where}: shape {list(shape)} of {dtype} needs "
                                   f"{count * _STORED[dtype][1]} bytes, data range holds {end - begin}")
        return TensorEntry(name, dtype, shape, si, begin, end)

    # ------------------------------------------------------------------
    def names(self) -> List[str]:
        return list(self.entries)

    def __contains__(self, name: str) -> bool:
        return name in self.entries

    def shape(self, name: str) -> Tuple[int, ...]:
        return self.entries[name].shape

    def stored_dtype(self, name: str) -> str:
        """The container's name of the element type ("BF16", "F32", ...)."""
        return self.entries[name].dtype

    def read(self, name: str) -> torch.Tensor:
        """The tensor in its kept dtype, on the CPU.  bfloat16, half-precision and 32-bit
        tensors are views of the mapped file; others are converted."""
        e = self.entries[name]
        stored, _ = _STORED[e.dtype]
        if e.end == e.begin:
            return torch.empty(e.shape, dtype=kept_dtype(e.dtype))
        buf = self._shards[e.shard].view(e.begin, e.end)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", UserWarning)     # the mapping is read-only; nothing writes to it
            t = torch.frombuffer(buf, dtype=stored).reshape(e.shape)
        keep = kept_dtype(e.dtype)
        if t.dtype == keep:
            return t
        if keep == torch.int32:
            from .loader import narrow_to_int32
            return narrow_to_int32(t.to(torch.int64) if t.dtype == torch.bool else t, name)
        return t.to(keep)


def write_safetensors(path: str, tensors: Mapping[str, torch.Tensor]) -> None:
    """Write one shard: 8-byte header length, JSON header, tensor bytes in the given order."""
    header = {}
    offset = 0
    items: List[Tuple[str, torch.Tensor]] = []
    for name, t in tensors.items():
        t = t.detach().cpu().contiguous()
        if t.dtype not in _WRITE_NAME:
            raise SafetensorsError(f"cannot store tensor {name!r} of dtype {t.dtype}")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _WRITE_NAME[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        items.append((name, t))
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for _, t in items:
            if t.numel():
                f.write(t.reshape(-1).view(torch.uint8).numpy())
