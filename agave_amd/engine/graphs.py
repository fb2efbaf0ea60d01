"""HIP graphs for decode steps.

A decode step launches some ten kernels per layer, each of them far shorter than the time the
host needs to launch it; recorded once into a HIP graph, the whole step is launched with one
call.  A graph is valid for one batch size and one bound on how many pages a sequence spans
(the attention kernels' split plan is fixed inside it); everything that changes from step to
step (tokens, positions, page tables) lives in one device buffer that is refilled before each
launch.  The first step of a kind runs eagerly (it sizes the workspace), the second one is
recorded, later ones are replayed.  At most ``max_graphs`` graphs are kept; when another kind
of step is to be recorded, the graph that has gone unused for longest makes room (a batch
whose requests end one by one passes through every batch size once and does not come back).

No memset node is recorded: nothing in the step clears memory.
"""
from __future__ import annotations

from collections import OrderedDict
from typing import Dict, Optional, Tuple

import torch


def span_bucket(span: int) -> int:
    """Pages a graph plans for: the next power of two, at least 4."""
    b = 4
    while b < span:
        b *= 2
    return b


class DecodeGraphs:
    def __init__(self, engine, max_graphs: int = 16):
        self.engine = engine
        self.max_graphs = max_graphs
        if max_graphs < 1:
            raise ValueError("max_graphs must be at least 1")
        self._seen: Dict[Tuple, int] = {}
        # least recently used first
        self._graphs: "OrderedDict[Tuple, Tuple[torch.cuda.CUDAGraph, Optional[torch.Tensor]]]" = OrderedDict()
        self.evicted = 0
        self._stamp = None

    def _valid_stamp(self):
        eng = self.engine
        return (eng.workspace.generation, eng.planner.buffer_generation)

    def run(self, step) -> Optional[torch.Tensor]:
        """Run a decode step whose wanted rows are all its rows; returns the logits."""
        eng = self.engine
        key = (step.n_seqs, step.fixed_span, tuple(t.shape[1] for t, _ in step.tables))
        if self._stamp != self._valid_stamp():
            self._graphs.clear()                 # a buffer moved: recorded addresses are stale
        entry = self._graphs.get(key)
        if entry is not None:
            self._graphs.move_to_end(key)
            entry[0].replay()
            return entry[1]
        count = self._seen.get(key, 0)
        self._seen[key] = count + 1
        if count == 0:
            return eng.model.forward(step)       # eager: loads libraries, sizes the workspace
        torch.cuda.synchronize(eng.device)       # nothing recorded is running when a graph is dropped or made
        while len(self._graphs) >= self.max_graphs:
            old, dropped = self._graphs.popitem(last=False)
            del dropped
            self._seen.pop(old, None)            # should its kind of step come back, it starts over
            self.evicted += 1
        stamp = self._valid_stamp()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = eng.model.forward(step)
        if self._valid_stamp() != stamp:
            # the workspace grew while recording: do not keep the graph, run the step eagerly
            return eng.model.forward(step)
        self._graphs[key] = (graph, logits)
        self._stamp = stamp
        graph.replay()
        return logits
