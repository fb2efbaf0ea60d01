"""One step: a batch of sequences that start together, with unequal lengths.

The first step of a batch brings every prompt whole, later steps one token per sequence.
A step runs only the tokens it is given, as one ragged batch (no padding token enters the
model), from the cache that earlier steps left, and returns the logits at the wanted places.

Reference: the reference has ``forward(one token)`` and ``prefill(one sequence)`` on a single
sequence (``src/models/gemma3.zig:331-368, 373-411``); positions of a chunk are
``base + t`` (``:430-432``), and only the last row's logits are computed (``:393-403``).
The batch, the slots and the choice of wanted rows are this engine's own.

Everything the kernels need to know about the step travels to the device as one block of
int32: the tokens, for every token its sequence and its position, the wanted rows, and for
every cache group one row of page ids per sequence with the page index its first column
stands for.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple, Union

import numpy as np
import torch

from ..cache import PAGE, KVCache, pages_in_reach

Want = Union[str, Sequence[Sequence[int]]]


class StepError(ValueError):
    pass


@dataclass
class Step:
    n_tokens: int
    n_seqs: int
    n_want: int
    slots: List[int]
    pos0: List[int]                 # length of each sequence before the step
    n_new: List[int]                # tokens each sequence brings
    cu: List[int]                   # prefix sums of the rows each sequence has in the step (host): n_new, and n_pad behind the last
    max_new: int
    max_len: int                    # longest sequence after the step
    tokens: torch.Tensor            # int32 [N] (device)
    tok_seq: torch.Tensor           # int32 [N]: index of the token's sequence in this step
    tok_pos: torch.Tensor           # int32 [N]: absolute position
    slots_dev: torch.Tensor         # int32 [B]
    pos0_dev: torch.Tensor          # int32 [B]
    cu_dev: torch.Tensor            # int32 [B + 1]
    want_rows: torch.Tensor         # int32 [n_want]: rows of the step whose logits are wanted
    tables: List[Tuple[torch.Tensor, torch.Tensor]]   # per cache group: (pages [B, width], base [B])
    bases_host: List[List[int]]     # per cache group: the host's copy of base
    cache: KVCache
    workspace: object = None
    fixed_span: Optional[int] = None    # a captured decode graph plans its splits for this many pages
    tables_start_at_reach: bool = False  # decode: column 0 of every table row is the first page the token reaches
    carry_dev: Optional[torch.Tensor] = None    # int32 [B]: rows of the previous step's sample that these tokens are
    floats_dev: Optional[torch.Tensor] = None   # float32 payload that travelled with the step (sampling parameters)
    n_pad: int = 0                               # rows behind the last sequence's tokens that belong to no request (see plan)

    def page_span(self, window: Optional[int]) -> int:
        """Most pages any sequence's last token of this step reaches back over."""
        if self.fixed_span is not None:
            span = self.fixed_span
            if window is not None:
                span = min(span, pages_in_reach(window, span * PAGE, 1))
            return max(1, span)
        span = 1
        for p0, n in zip(self.pos0, self.n_new):
            p = p0 + n - 1
            lo = max(0, p - window + 1) if window is not None else 0
            span = max(span, p // PAGE - lo // PAGE + 1)
        return span

    @property
    def is_decode(self) -> bool:
        return self.max_new == 1

    def base_of(self, base: torch.Tensor) -> Optional[List[int]]:
        """The host's copy of a group's ``base`` tensor (one of ``tables``), for checks before a launch."""
        for (_, dev), host in zip(self.tables, self.bases_host):
            if dev is base:
                return host
        return None


def resolve_want(want: Want, n_new: Sequence[int]) -> List[List[int]]:
    if isinstance(want, str):
        if want == "last":
            return [[n - 1] for n in n_new]
        if want == "all":
            return [list(range(n)) for n in n_new]
        if want == "none":
            return [[] for _ in n_new]
        raise StepError(f"want must be 'last', 'all', 'none' or lists of places, got {want!r}")
    if len(want) != len(n_new):
        raise StepError(f"want lists {len(want)} sequences, the step has {len(n_new)}")
    out = []
    for i, (w, n) in enumerate(zip(want, n_new)):
        w = [int(x) for x in w]
        for x in w:
            if not (0 <= x < n):
                raise StepError(f"sequence {i}: wanted place {x} is outside its {n} tokens")
        out.append(w)
    return out


def split_pieces(n_new: Sequence[int], piece: int) -> List[List[int]]:
    """How a step whose sequences bring ``n_new[i]`` tokens runs when no sequence may bring more
    than ``piece`` at a time: while a sequence has more than ``piece`` tokens left, those that do
    run their next ``piece`` tokens together; the last step holds every sequence with what it
    has left (at least one token, at most ``piece``).  Returns the token counts of each step in
    turn (0: the sequence takes no part in it).  The reference feeds a prompt in chunks the same
    way, one sequence at a time (``src/models/gemma3.zig:385-391``)."""
    if piece < 1:
        raise StepError("a step's pieces hold at least one token")
    left = [int(n) for n in n_new]
    out: List[List[int]] = []
    while max(left) > piece:
        now = [piece if n > piece else 0 for n in left]
        out.append(now)
        left = [n - k for n, k in zip(left, now)]
    out.append(left)
    return out


class StepPlanner:
    """Turns (slots, tokens, want) into a :class:`Step`: checks the request, takes cache
    pages, and uploads the step's description in one copy."""

    def __init__(self, cache: KVCache, vocab_size: int, device: torch.device, workspace=None):
        self.cache = cache
        self.workspace = workspace
        self.vocab_size = vocab_size
        self.device = device
        self._hosts: List[Optional[torch.Tensor]] = [None, None]   # two pinned buffers in turn: a step may be
        self._copied: List[Optional[torch.cuda.Event]] = [None, None]  # planned while the one before still waits
        self._turn = 0
        self._dev: Optional[torch.Tensor] = None
        self.fixed_width: Optional[List[int]] = None   # table widths pinned for graph capture
        self.buffer_generation = 0   # changes when the device buffer of the step's description moves

    def _buffers(self, n: int) -> torch.Tensor:
        """The pinned host buffer of this turn, at least ``n`` int32 long, free to be written."""
        self._turn ^= 1
        t = self._turn
        if self._copied[t] is not None:
            self._copied[t].synchronize()          # its last upload has left it
        host = self._hosts[t]
        if host is None or host.numel() < n:
            cap = max(n, 4096) if host is None else max(n, 2 * host.numel())
            self._hosts[t] = host = torch.empty(cap, dtype=torch.int32, pin_memory=True)
        if self._dev is None or self._dev.numel() < host.numel():
            self._dev = torch.empty(host.numel(), dtype=torch.int32, device=self.device)
            self.buffer_generation += 1
        return host

    def plan(self, slots: Sequence[int], tokens: Sequence[Sequence[int]], want: Want = "last",
             decode_widths: Optional[List[int]] = None, carry: Optional[Sequence[int]] = None,
             floats: Optional[np.ndarray] = None, pad_to: int = 0) -> Step:
        """``decode_widths``: table widths to use if this turns out to be a decode step (one token per
        sequence), so that all decode steps of a batch size have the same layout on the device.
        ``carry``: one index per sequence into what the previous step sampled (the tokens given
        are placeholders then); ``floats``: float32 values that travel in the same upload.  Both
        lie behind everything else, so they do not move what a recorded graph reads.
        ``pad_to`` (a step of one sequence; a divisor of the page's length): rows are added behind
        the sequence's tokens until it ends at a multiple of ``pad_to``, so that every step that
        ends in the same stretch has the same shape and can be replayed as one recorded graph.
        The added rows carry token 0 at the positions that follow and run through the model like
        the others (``cu`` counts them, ``n_new`` and the wanted rows do not, ``n_pad`` says how
        many they are); they belong to no request: the sequence's length stays the real one,
        attention never looks at a later position, and the keys and values that the rows leave in
        the unused places of the sequence's last page are
        overwritten by the tokens that come to stand there before anything reads them."""
        if len(slots) != len(tokens) or len(slots) == 0:
            raise StepError("a step needs as many token lists as slots, and at least one")
        n_new = [len(t) for t in tokens]
        if min(n_new) < 1:
            raise StepError("every sequence of a step brings at least one token")
        flat = np.fromiter((int(x) for t in tokens for x in t), dtype=np.int64, count=sum(n_new))
        if flat.size and (flat.min() < 0 or flat.max() >= self.vocab_size):
            bad = int(flat[(flat < 0) | (flat >= self.vocab_size)][0])
            raise StepError(f"token id {bad} is outside the vocabulary of {self.vocab_size}")
        wanted = resolve_want(want, n_new)
        pos0, plans = self.cache.plan_step(list(slots), n_new)

        b, n_real = len(slots), int(flat.size)
        cu = [0]
        for x in n_new:
            cu.append(cu[-1] + x)
        want_rows = [cu[i] + x for i, w in enumerate(wanted) for x in w]
        n_pad = 0
        if pad_to:
            if b != 1 or PAGE % pad_to:
                raise StepError("only a step of one sequence is padded, and only within its last page")
            n_pad = (-(pos0[0] + n_new[0])) % pad_to
        n = n_real + n_pad
        rows_of = list(n_new)
        rows_of[-1] += n_pad                 # the added rows follow the last sequence's tokens and positions
        cu = list(cu)
        cu[-1] += n_pad                      # to the kernels they are rows of that sequence like the others
        widths = []
        fixed = decode_widths if (decode_widths is not None and max(n_new) == 1) else self.fixed_width
        for gi, p in enumerate(plans):
            w = max(len(r) for r in p.rows)
            if fixed is not None and w <= fixed[gi]:
                w = fixed[gi]
            widths.append(w)
        n_carry = len(carry) if carry is not None else 0
        n_floats = int(floats.size) if floats is not None else 0
        if carry is not None and n_carry != b:
            raise StepError("carry needs one index per sequence")
        total = 3 * n + 3 * b + 1 + len(want_rows) + sum(b + b * w for w in widths) + n_carry + n_floats
        host_t = self._buffers(total)
        host = host_t.numpy()
        off = 0

        def put(values, count) -> Tuple[int, int]:
            nonlocal off
            host[off:off + count] = values
            span = (off, off + count)
            off += count
            return span

        s_tok = put(np.concatenate([flat, np.zeros(n_pad, dtype=np.int64)]) if n_pad else flat, n)
        s_seq = put(np.repeat(np.arange(b, dtype=np.int32), rows_of), n)
        s_pos = put(np.concatenate([np.arange(p, p + k, dtype=np.int32) for p, k in zip(pos0, rows_of)]), n)
        s_slots = put(np.asarray(slots, dtype=np.int32), b)
        s_pos0 = put(np.asarray(pos0, dtype=np.int32), b)
        s_cu = put(np.asarray(cu, dtype=np.int32), b + 1)
        s_want = put(np.asarray(want_rows, dtype=np.int32), len(want_rows))
        s_tables = []
        for p, w in zip(plans, widths):
            s_base = put(np.asarray(p.base, dtype=np.int32), b)
            tab = np.full((b, w), -1, dtype=np.int32)
            for i, r in enumerate(p.rows):
                tab[i, :len(r)] = r
            s_tables.append((put(tab.reshape(-1), b * w), s_base, w))
        s_carry = put(np.asarray(carry, dtype=np.int32), n_carry) if carry is not None else None
        s_floats = None
        if floats is not None:
            s_floats = put(np.ascontiguousarray(floats, dtype=np.float32).reshape(-1).view(np.int32), n_floats)
        assert off == total
        self._dev[:total].copy_(host_t[:total], non_blocking=True)
        self._copied[self._turn] = torch.cuda.Event()
        self._copied[self._turn].record()
        d = self._dev

        def view(span):
            return d[span[0]:span[1]]

        return Step(
            n_tokens=n, n_seqs=b, n_want=len(want_rows), slots=list(slots), pos0=pos0, n_new=n_new, cu=cu,
            max_new=max(n_new), max_len=max(p + k for p, k in zip(pos0, n_new)),
            tokens=view(s_tok), tok_seq=view(s_seq), tok_pos=view(s_pos), slots_dev=view(s_slots),
            pos0_dev=view(s_pos0), cu_dev=view(s_cu), want_rows=view(s_want),
            tables=[(view(t).view(b, w), view(sb)) for t, sb, w in s_tables],
            bases_host=[list(p.base) for p in plans], cache=self.cache,
            workspace=self.workspace, tables_start_at_reach=(max(n_new) == 1),
            carry_dev=view(s_carry) if s_carry is not None else None,
            floats_dev=view(s_floats).view(torch.float32) if s_floats is not None else None, n_pad=n_pad)

    def commit(self, step: Step) -> None:
        self.cache.commit_step(step.slots, step.n_new)
