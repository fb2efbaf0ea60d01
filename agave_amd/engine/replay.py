"""Trace replay over the engine's own step function (used by ``bin/trace_run``).

The nearest thing in the reference is its golden harness, which spawns the command line and
compares text (``tests/models/golden_harness.zig:152-287``); this replays token ids and hands
back logits instead, so that a position's logits can be compared however the tokens were cut
into steps and batches.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import numpy as np

from ..cache import PAGE
from .engine import Engine


class Replay:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int):
        pages = (int(max_tokens) + PAGE - 1) // PAGE
        # every live request holds at least one page, so there are never more requests than pages
        self.engine = Engine.from_folder(model_dir, dtype=dtype, max_slots=pages,
                                         max_context=pages * PAGE, cache_tokens=pages * PAGE)
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
