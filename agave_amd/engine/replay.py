"""Trace replay over the engine's own step function (used by ``bin/trace_run``).

The nearest thing in the reference is its golden harness, which spawns the command line and
compares text (``tests/models/golden_harness.zig:152-287``); this replays token ids and hands
back logits instead, so that a position's logits can be compared however the tokens were cut
into steps and batches.

Two ways in: steps given one by one (:meth:`Replay.run_step`), and whole requests with a way of
cutting them (:func:`plan_steps`, :meth:`Replay.run_requests`):

``whole``    each request alone, all its tokens in one step;
``tail32``   each request alone: all but the last 32 tokens in one step, then those one by one;
``batched``  batches of requests that start together: the first step brings each request's
             prompt (``prompt`` tokens of it, default all but its last 32), then one token each
             until a request's tokens are used up; it then leaves the batch, and one batch runs
             after another, so that slots and pages are used again.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from ..cache import PAGE
from .engine import Engine

MODES = ("whole", "tail32", "batched")
TAIL = 32


def plan_steps(mode: str, requests: Sequence[dict], batch_size: int = 0) -> Tuple[List[dict], Dict[str, List[Tuple[int, int]]]]:
    """Cut ``requests`` (dicts with ``id``, ``tokens`` and, for ``batched``, optionally ``prompt``
    and ``batch``) into steps.  Returns (step records in the form :meth:`Replay.run_step` takes,
    with every fed position wanted; where[id] = for each of the request's positions the
    (step, row among that step's wanted rows) that holds its logits).  In ``batched`` mode requests
    with the same ``batch`` value run together; without it, ``batch_size`` (0: all) in the order given."""
    if mode not in MODES:
        raise ValueError(f"unknown mode {mode!r}; known: {', '.join(MODES)}")
    reqs = []
    for r in requests:
        toks = [int(t) for t in r["tokens"]]
        if not toks:
            raise ValueError(f"request {r.get('id')!r} has no tokens")
        reqs.append((str(r["id"]), toks, r))
    if len({rid for rid, _, _ in reqs}) != len(reqs):
        raise ValueError("request ids must differ")
    if mode == "batched":
        groups: Dict[object, List[int]] = {}
        for i, (_, _, r) in enumerate(reqs):
            key = r["batch"] if "batch" in r else (i // batch_size if batch_size > 0 else 0)
            groups.setdefault(key, []).append(i)
        batches = list(groups.values())
    else:
        batches = [[i] for i in range(len(reqs))]
    records: List[dict] = []
    where: Dict[str, List[Tuple[int, int]]] = {rid: [] for rid, _, _ in reqs}
    for members in batches:
        used = {}
        for i in members:
            rid, toks, r = reqs[i]
            if mode == "whole":
                used[i] = len(toks)
            elif mode == "tail32" or "prompt" not in r:
                used[i] = len(toks) - min(TAIL, len(toks) - 1)
            else:
                used[i] = max(1, min(int(r["prompt"]), len(toks)))
        live = list(members)
        first = True
        while live:
            entries, row = [], 0
            for i in live:
                rid, toks, _ = reqs[i]
                n = used[i] if first else 1
                lo = 0 if first else used[i]
                entries.append({"id": rid, "tokens": toks[lo:lo + n], "want": list(range(n))})
                where[rid] += [(len(records), row + k) for k in range(n)]
                row += n
                if not first:
                    used[i] += 1
            first = False
            ended = [i for i in live if used[i] >= len(reqs[i][1])]
            records.append({"step": len(records), "entries": entries, "end": [reqs[i][0] for i in ended]})
            live = [i for i in live if i not in ended]
    return records, where


def tokens_held(records: Sequence[dict]) -> int:
    """The most tokens that live requests hold at any time over these steps, each request's count
    rounded up to a multiple of 64: what the cache must be sized for."""
    held: Dict[str, int] = {}
    most = 0
    for rec in records:
        for e in rec["entries"]:
            held[str(e["id"])] = held.get(str(e["id"]), 0) + len(e["tokens"])
        most = max(most, sum(-(-n // PAGE) * PAGE for n in held.values()))
        for rid in rec.get("end", []):
            held.pop(str(rid), None)
    return most


class Replay:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int):
        pages = (int(max_tokens) + PAGE - 1) // PAGE
        # every live request holds at least one page, so there are never more requests than pages
        self.engine = Engine.from_folder(model_dir, dtype=dtype, max_slots=pages,
                                         max_context=pages * PAGE, cache_tokens=pages * PAGE, will_sample=False)
        self.slot_of: Dict[str, int] = {}

    def run_step(self, entries: Sequence[dict], end: Sequence[str]) -> Optional[np.ndarray]:
        """Run one step; float32 logits [wanted, vocab] on the host, or None."""
        out = None
        if entries:
            slots, tokens, want = [], [], []
            for e in entries:
                rid = str(e["id"])
                if rid not in self.slot_of:
                    self.slot_of[rid] = self.engine.alloc_slot()
                slots.append(self.slot_of[rid])
                tokens.append([int(t) for t in e["tokens"]])
                want.append([int(w) for w in e.get("want", [])])
            logits = self.engine.step(slots, tokens, want)
            if logits is not None:
                out = logits.cpu().numpy()
        for rid in end:
            slot = self.slot_of.pop(str(rid), None)
            if slot is not None:
                self.engine.free_slot(slot)
        return out

    def run_requests(self, mode: str, requests: Sequence[dict], batch_size: int = 0,
                     on_step=None) -> Dict[str, np.ndarray]:
        """Feed whole requests, cut as ``mode`` says; {id: float32 logits [its positions, vocab]}."""
        records, where = plan_steps(mode, requests, batch_size)
        vocab = self.engine.vocab_size
        out = {rid: np.empty((len(places), vocab), dtype=np.float32) for rid, places in where.items()}
        at = {rid: 0 for rid in where}
        for rec in records:
            logits = self.run_step(rec["entries"], rec["end"])
            row = 0
            for e in rec["entries"]:
                n = len(e["want"])
                rid = str(e["id"])
                out[rid][at[rid]:at[rid] + n] = logits[row:row + n]
                at[rid] += n
                row += n
            if on_step is not None:
                on_step(rec["step"])
        return out
