"""HIP graphs for decode steps, and for short prompts of one sequence.

A decode step launches some ten kernels per layer, each of them far shorter than the time the
host needs to launch it; recorded once into a HIP graph, the whole step is launched with one
call.  A graph is valid for one batch size and one bound on how many pages a sequence spans
(the attention kernels' split plan is fixed inside it); everything that changes from step to
step (tokens, positions, page tables) lives in one device buffer that is refilled before each
launch.  The first step of a kind runs eagerly (it sizes the workspace), the second one is
recorded, later ones are replayed.  At most ``max_graphs`` graphs are kept; when another kind
of step is to be recorded, the graph that has gone unused for longest makes room (a batch
whose requests end one by one passes through every batch size once and does not come back).

A short prompt of one sequence (up to ``PROMPT_GRAPH_TOKENS`` rows) is recorded too: the planner
pads it until it ends at a multiple of ``PROMPT_GRAPH_PAD`` positions, so every prompt that starts
at the same position and ends in the same stretch is the same step to the device, down to the
attention kernel's list of items, which is made for the padded length and kept with the graph.
Such a prompt's 280 launches take the host longer than they take the GPU; replayed, the step
takes what its kernels take.  Longer prompts are not recorded: there the host keeps ahead of the
GPU, and the padding would cost more than the launches.

No memset node is recorded: nothing in the step clears memory.
"""
from __future__ import annotations

from collections import OrderedDict
from typing import Dict, Optional, Tuple

import torch


PROMPT_GRAPH_TOKENS = 128      # rows (with padding) up to which a prompt of one sequence is replayed as a graph
PROMPT_GRAPH_PAD = 16          # such a prompt is padded until it ends at a multiple of this many positions


def span_bucket(span: int) -> int:
    """Pages a graph plans for: the next power of two, at least 4."""
    b = 4
    while b < span:
        b *= 2
    return b


class DecodeGraphs:
    def __init__(self, engine, max_graphs: int = 32):
        self.engine = engine
        self.max_graphs = max_graphs
        if max_graphs < 1:
            raise ValueError("max_graphs must be at least 1")
        self._seen: Dict[Tuple, int] = {}
        # least recently used first
        self._graphs: "OrderedDict[Tuple, Tuple[torch.cuda.CUDAGraph, Optional[torch.Tensor]]]" = OrderedDict()
        self._plans: Dict[Tuple, dict] = {}      # prompt steps: the attention kernels' host-made plans, by kind of step
        self.evicted = 0
        self._stamp = None

    def _valid_stamp(self):
        eng = self.engine
        return (eng.workspace.generation, eng.planner.buffer_generation)

    def run(self, step) -> Optional[torch.Tensor]:
        """Run a decode step whose wanted rows are all its rows; returns the logits."""
        return self._run((step.n_seqs, step.fixed_span, tuple(t.shape[1] for t, _ in step.tables)), step)

    def run_prompt(self, step) -> Optional[torch.Tensor]:
        """Run a step of one sequence that the planner padded to a fixed multiple of rows and that
        wants its last real row; returns the logits."""
        key = ("prompt", step.n_tokens, step.pos0[0], tuple(t.shape[1] for t, _ in step.tables))
        # what the attention kernels make of the step's shape on the host (their lists of items) is the
        # same for every step of this kind: made by the first one, kept here, and handed to the later
        # ones, so that recording finds it on the device already
        if key not in self._plans and len(self._plans) >= 4 * self.max_graphs:
            # kinds of step that came once and never again (prompts that start at odd positions)
            for k in [k for k in self._plans if k not in self._graphs]:
                del self._plans[k]
                self._seen.pop(k, None)
        plans = self._plans.setdefault(key, {})
        step.__dict__["_prefill_items"] = plans
        return self._run(key, step)

    def _run(self, key, step) -> Optional[torch.Tensor]:
        eng = self.engine
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
            self._plans.pop(old, None)
            self.evicted += 1
        stamp, made = self._valid_stamp(), eng.workspace.allocations
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = eng.model.forward(step)
        if self._valid_stamp() != stamp or eng.workspace.allocations != made:
            # the workspace made or replaced a buffer while recording: do not keep the graph, run the
            # step eagerly (the kind's next step is recorded with every buffer in place)
            self._seen[key] = 1
            return eng.model.forward(step)
        self._graphs[key] = (graph, logits)
        self._stamp = stamp
        graph.replay()
        return logits
