"""The cache as the engine sees it: slots, key/value pages per group of layers, and
fixed-size per-sequence state.

A *memory* is what one entry of the model's run order reads and appends to (one layer's
keys and values, unless two entries share it).  Memories whose mixers need the same thing
(all keys or a window of them, the same number of kv heads and head size) form a group with
storage and a page pool of its own:

    K[memory, page, kv head, 64, head_dim]       V[memory, page, kv head, head_dim, 64]

(V is stored transposed inside a page so that the matrix cores read it along the keys.)
All memories of a group use the same page ids, so there is one table per group and step.
Mixers with state of fixed size get ``state[memory][slot, ...]``, zeroed when a slot is
taken.  Gemma 3 has none; the store exists for mixers that do.

Reference: ``PagedKvCache`` / ``SeqBlockTable`` (``src/kvcache/manager.zig:76-185``),
``resetKvCache`` (``src/models/model.zig:474-485``), ``KVCacheFull``
(``src/models/gemma3.zig:332``).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .pages import PAGE, CacheError, GroupKey, GroupPages, OutOfPages, SlotTable


@dataclass(frozen=True)
class StateNeed:
    """Fixed-size state of one memory: ``shape`` per sequence."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class GroupPlan:
    """One group's part of a step, on the host: per sequence the first page index of its
    table row and the row itself."""
    base: List[int]
    rows: List[List[int]]


class KVCache:
    def __init__(self, kv_needs: Dict[int, GroupKey], state_needs: Dict[int, StateNeed], max_slots: int,
                 pages_per_group: Dict[GroupKey, int], dtype: torch.dtype, device: Optional[torch.device],
                 max_context: int):
        """``kv_needs``: memory id -> what its mixer needs; ``pages_per_group``: pool sizes.
        ``device`` None keeps only the bookkeeping (tests without a GPU)."""
        self.max_slots = max_slots
        self.max_context = max_context
        self.dtype = dtype
        self.device = device
        self.slots = SlotTable(max_slots)
        self.group_keys: List[GroupKey] = []
        self.group_of_memory: Dict[int, int] = {}
        self.index_in_group: Dict[int, int] = {}
        members: List[List[int]] = []
        for mem in sorted(kv_needs):
            key = kv_needs[mem]
            if key not in self.group_keys:
                self.group_keys.append(key)
                members.append([])
            g = self.group_keys.index(key)
            self.group_of_memory[mem] = g
            self.index_in_group[mem] = len(members[g])
            members[g].append(mem)
        self.groups: List[GroupPages] = [GroupPages(k, pages_per_group[k], max_slots) for k in self.group_keys]
        self.k_store: List[Optional[torch.Tensor]] = []
        self.v_store: List[Optional[torch.Tensor]] = []
        # bfloat16 groups whose head size is a multiple of 16 (up to 256) keep their pages in the
        # matrix cores' tile order; the others row by row
        self.packed: List[bool] = [dtype == torch.bfloat16 and k.head_dim % 16 == 0 and k.head_dim <= 256
                                   for k in self.group_keys]
        for key, mems, packed in zip(self.group_keys, members, self.packed):
            n = pages_per_group[key]
            hd_k = (key.head_dim + 31) // 32 * 32 if packed else key.head_dim
            if device is None:
                self.k_store.append(None)
                self.v_store.append(None)
            else:
                self.k_store.append(torch.zeros((len(mems), n, key.n_kv_heads, PAGE, hd_k), dtype=dtype, device=device))
                self.v_store.append(torch.zeros((len(mems), n, key.n_kv_heads, key.head_dim, PAGE), dtype=dtype, device=device))
        self.state_needs = dict(state_needs)
        self.state: Dict[int, Optional[torch.Tensor]] = {}
        for mem, need in state_needs.items():
            self.state[mem] = None if device is None else torch.zeros((max_slots,) + tuple(need.shape), dtype=need.dtype, device=device)

    # ------------------------------------------------------------------ slots
    def alloc_slot(self) -> int:
        s = self.slots.alloc()
        for t in self.state.values():
            if t is not None:
                t[s].zero_()
        return s

    def free_slot(self, slot: int) -> None:
        self.slots.check(slot)
        for g in self.groups:
            g.release(slot)
        self.slots.free(slot)

    def length(self, slot: int) -> int:
        self.slots.check(slot)
        return self.slots.length[slot]

    # ------------------------------------------------------------------ steps
    def plan_step(self, slots: Sequence[int], n_new: Sequence[int]) -> Tuple[List[int], List[GroupPlan]]:
        """Check and prepare a step that appends ``n_new[i]`` positions to ``slots[i]``.
        Nothing is changed unless the whole step fits.  Returns the sequences' lengths
        before the step and one plan per group."""
        if len(set(slots)) != len(slots):
            raise CacheError("a slot appears twice in one step")
        pos0 = []
        for s, n in zip(slots, n_new):
            self.slots.check(s)
            if n < 1:
                raise CacheError("a step brings at least one token per sequence")
            cur = self.slots.length[s]
            if cur + n > self.max_context:
                raise CacheError(f"slot {s}: {cur} + {n} positions exceed the context of {self.max_context}")
            pos0.append(cur)
        # all groups and sequences must fit before anything is taken
        for g in self.groups:
            need = 0
            for s, p0, n in zip(slots, pos0, n_new):
                held = g.held(s)
                need += sum(1 for i in range(p0 // PAGE, (p0 + n - 1) // PAGE + 1) if i not in held)
            if need > g.pool.n_free:
                raise OutOfPages(f"step needs {need} more cache pages of group {g.key}, "
                                 f"{g.pool.n_free} of {g.pool.n_pages} are free")
        plans = []
        for g in self.groups:
            base, rows = [], []
            for s, p0, n in zip(slots, pos0, n_new):
                b, r = g.plan(s, p0, n)
                base.append(b)
                rows.append(r)
            plans.append(GroupPlan(base, rows))
        return pos0, plans

    def check_pieces(self, slots: Sequence[int], pieces: Sequence[Sequence[int]]) -> None:
        """Raise, changing nothing, unless a step that is run as several steps one after another
        fits as a whole.  ``pieces[j][i]`` is the number of tokens that ``slots[i]`` brings in
        the j-th of them (0: it takes no part).  Every sequence must stay within the context, and
        in every group the pages held at the fullest moment must be there: a windowed group
        gives pages back between the pieces, a group that needs all keys does not."""
        if len(set(slots)) != len(slots):
            raise CacheError("a slot appears twice in one step")
        lengths = []
        for i, s in enumerate(slots):
            self.slots.check(s)
            cur = self.slots.length[s]
            total = sum(int(p[i]) for p in pieces)
            if cur + total > self.max_context:
                raise CacheError(f"slot {s}: {cur} + {total} positions exceed the context of {self.max_context}")
            lengths.append(cur)
        for g in self.groups:
            held = [set(g.held(s)) for s in slots]
            there = g.pool.n_free + sum(len(h) for h in held)
            lens = list(lengths)
            for piece in pieces:
                for i, n in enumerate(piece):
                    if n > 0:
                        held[i].update(range(lens[i] // PAGE, (lens[i] + n - 1) // PAGE + 1))
                need = sum(len(h) for h in held)
                if need > there:
                    raise OutOfPages(f"step needs {need - there} more cache pages of group {g.key} than the "
                                     f"{g.pool.n_free} that are free of {g.pool.n_pages}")
                for i, n in enumerate(piece):
                    if n > 0:
                        lens[i] += n
                        keep_from = g._first_needed(lens[i])
                        held[i] = {x for x in held[i] if x >= keep_from}

    def commit_step(self, slots: Sequence[int], n_new: Sequence[int]) -> None:
        for s, n in zip(slots, n_new):
            self.slots.length[s] += n
            for g in self.groups:
                g.commit(s, self.slots.length[s])

    # ------------------------------------------------------------------ storage
    def pages_of(self, memory: int) -> Tuple[torch.Tensor, torch.Tensor, bool]:
        """(K pages, V pages, whether they are in the matrix cores' tile order) of one memory."""
        g, i = self.group_of_memory[memory], self.index_in_group[memory]
        return self.k_store[g][i], self.v_store[g][i], self.packed[g]

    def bytes(self) -> int:
        total = 0
        for t in self.k_store + self.v_store + list(self.state.values()):
            if t is not None:
                total += t.numel() * t.element_size()
        return total
