"""The generation loop above the step function: batches of unequal prompts, stop tokens,
sequences that end earlier, and as many batches one after another as there are requests.

Reference (one sequence): ``generateAndPrintInner`` (``src/main.zig:2118-2461``): the first
token comes from the prompt's last logits (``:2290-2294``), then up to ``max_tokens - 1``
further steps (``:2342``); the repeat penalty covers every id generated so far (``:2350-2352``);
an end-of-generation id stops the sequence and is not emitted (``:2366-2369``); a full cache
ends it too (``KVCacheFull``, ``src/models/gemma3.zig:332``).  Another thread may cancel the
call (the reference's ``cancelled`` flag, looked at between layers: ``src/models/gemma3.zig:141,
342``; here between steps): a backend with ``cancel_requested()`` is asked before every step, and
a cancelled call returns what it has, every unfinished request with the reason "cancelled".  The
reference's "halt after six
equal tokens" (``src/main.zig:2400-2407``) changes outputs and is not taken over.

The loop's decisions need no GPU: it talks to a *backend* with ``max_context``, ``max_slots``,
``alloc_slot()``, ``free_slot(slot)`` and ``step_sample(slots, tokens, rows) -> token ids``;
the engine is one, the tests use a fake.

A backend that also has ``launch_step(slots, tokens | None, rows, carry)`` and
``finish_step(handle)`` is driven one step ahead: the next step is launched, with its tokens
taken on the device from what the running step samples, before the running step's tokens are
read.  The host's work then hides behind the GPU's.  A sequence that turns out to have
stopped has run one step too many; that step's token for it is dropped and its slot is given
back once the step has ended.  Nothing a request gets depends on this.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Union

import numpy as np

from ..sampling import GenerationResult, SamplingParams


@dataclass
class RowSampling:
    """What the sampler needs for one sequence of a step."""
    temperature: float
    top_k: int
    top_p: float
    repeat_penalty: float
    u: float                     # uniform draw in [0, 1) of this request's own stream
    generated: List[int]         # ids generated so far (for the repeat penalty)
    logprob: bool = False        # the drawn token's log-probability is wanted


@dataclass
class GenerationStats:
    """Counters in the reference's terms (``src/display.zig:143-163, 702-744``)."""
    prefill_tokens: int = 0
    prefill_ms: float = 0.0
    tokens: int = 0              # generated tokens of all requests
    gen_ms: float = 0.0          # decode steps only
    decode_tokens: int = 0       # tokens produced by decode steps
    batches: int = 0

    @property
    def tok_per_sec(self) -> float:
        return self.decode_tokens / (self.gen_ms / 1e3) if self.gen_ms > 0 else 0.0

    @property
    def prefill_tok_per_sec(self) -> float:
        return self.prefill_tokens / (self.prefill_ms / 1e3) if self.prefill_ms > 0 else 0.0


def generate(backend, prompts: Sequence[Sequence[int]],
             params: Union[SamplingParams, Sequence[SamplingParams]] = SamplingParams(),
             eos_ids: Sequence[int] = (), max_batch: Optional[int] = None,
             stats: Optional[GenerationStats] = None) -> List[GenerationResult]:
    """Generate for every prompt (lists of token ids).  Requests run in batches of at most
    ``max_batch`` (default: the backend's slots), in the order given, one batch after another;
    a request's result does not depend on the others."""
    n = len(prompts)
    plist = [params] * n if isinstance(params, SamplingParams) else list(params)
    if len(plist) != n:
        raise ValueError(f"{len(plist)} sampling parameter sets for {n} prompts")
    max_batch = int(max_batch or backend.max_slots)
    if max_batch < 1 or max_batch > backend.max_slots:
        raise ValueError(f"max_batch must be in 1..{backend.max_slots}")
    stats = stats if stats is not None else GenerationStats()
    clock_seed = time.time_ns() & 0x7FFFFFFF
    results = [GenerationResult(i, len(p)) for i, p in enumerate(prompts)]
    rngs = [np.random.default_rng([p.seed if p.seed is not None else clock_seed, i]) for i, p in enumerate(plist)]
    stops = [set() if p.ignore_eos else (set(int(x) for x in eos_ids) | set(p.stop_ids)) for p in plist]

    queue = []
    for i, p in enumerate(prompts):
        if len(p) == 0:
            raise ValueError(f"prompt {i} is empty (give at least the begin-of-sequence id)")
        if len(p) > backend.max_context:
            results[i].finish_reason = "context"        # the prompt alone does not fit a slot
        else:
            queue.append(i)

    def row(i: int) -> RowSampling:
        p = plist[i]
        u = float(rngs[i].random(dtype=np.float32)) if p.temperature > 0 else 0.0
        return RowSampling(p.temperature, p.top_k, p.top_p, p.repeat_penalty, u, results[i].tokens, p.logprobs)

    ahead = hasattr(backend, "launch_step") and all(p.repeat_penalty == 1.0 for p in plist)
    cancel_requested = getattr(backend, "cancel_requested", lambda: False)

    def settle(i: int, tok: int, logprob: Optional[float] = None) -> None:
        """Book the token request i drew; sets its finish reason if it ends here."""
        r = results[i]
        if tok in stops[i]:
            r.finish_reason = "stop"                      # the end token is not emitted
        else:
            r.tokens.append(tok)
            if plist[i].logprobs and logprob is not None:
                r.logprobs.append(logprob)
            stats.tokens += 1
            if len(r.tokens) >= plist[i].max_tokens:
                r.finish_reason = "length"
            elif r.prompt_tokens + len(r.tokens) > backend.max_context:
                r.finish_reason = "context"               # no room to feed this token

    while queue:
        if cancel_requested():
            break
        batch, queue = queue[:max_batch], queue[max_batch:]
        stats.batches += 1
        slots = {i: backend.alloc_slot() for i in batch}
        live = list(batch)
        feed = [list(prompts[i]) for i in live]
        first = True
        try:
            if not ahead:
                while live and not cancel_requested():
                    t0 = time.perf_counter()
                    sampled = backend.step_sample([slots[i] for i in live], feed, [row(i) for i in live])
                    ms = (time.perf_counter() - t0) * 1e3
                    if first:
                        stats.prefill_tokens += sum(len(f) for f in feed)
                        stats.prefill_ms += ms
                    else:
                        stats.gen_ms += ms
                        stats.decode_tokens += len(live)
                    first = False
                    nxt = []
                    lps = getattr(backend, "last_logprobs", None) or [None] * len(live)
                    for i, tok, lp in zip(live, sampled, lps):
                        settle(i, int(tok), lp)
                        if results[i].finish_reason:
                            backend.free_slot(slots.pop(i))               # given back at once
                        else:
                            nxt.append(i)
                    live = nxt
                    feed = [[results[i].tokens[-1]] for i in live]
                continue
            # one step ahead: `running` is the step under way over the requests `live`, some of which
            # may have ended with the token before (this is then their step too many)
            t0 = time.perf_counter()
            running = backend.launch_step([slots[i] for i in live], feed, [row(i) for i in live], None)
            stats.prefill_tokens += sum(len(f) for f in feed)
            while True:
                # who goes on unless the running step draws an end token: known beforehand
                on = [i for i in live if not results[i].finish_reason and not cancel_requested()
                      and len(results[i].tokens) + 1 < plist[i].max_tokens
                      and results[i].prompt_tokens + len(results[i].tokens) + 1 <= backend.max_context]
                following = None
                if on:
                    following = backend.launch_step([slots[i] for i in on], None, [row(i) for i in on],
                                                    [live.index(i) for i in on])
                sampled = backend.finish_step(running)
                ms = (time.perf_counter() - t0) * 1e3
                t0 = time.perf_counter()
                if first:
                    stats.prefill_ms += ms
                else:
                    stats.gen_ms += ms
                lps = getattr(backend, "last_logprobs", None) or [None] * len(live)
                for i, tok, lp in zip(live, sampled, lps):
                    if results[i].finish_reason:
                        backend.free_slot(slots.pop(i))       # ended a step ago; no step uses its slot now
                        continue
                    settle(i, int(tok), lp)
                    if not first:
                        stats.decode_tokens += 1
                    if results[i].finish_reason and i not in on:
                        backend.free_slot(slots.pop(i))       # not part of the step that is under way
                first = False
                if following is None:
                    break
                live, running = on, following
        finally:
            for s in slots.values():
                backend.free_slot(s)
    if cancel_requested():
        for r in results:
            if not r.finish_reason:
                r.finish_reason = "cancelled"
        # The call that a request to cancel ends also uses it up (the reference's owner resets the
        # flag between requests, src/models/model.zig:315-317).  It is not cleared on entry: a
        # request that arrives just before the call starts ends that call before its first step.
        if hasattr(backend, "clear_cancel"):
            backend.clear_cancel()
    return results
