"""Sampling options with the reference's names, meanings and defaults.

Reference: ``src/main.zig:333-339`` (``-n/--max-tokens`` 512, ``-t/--temperature`` 0,
``--top-p`` 1.0, ``--top-k`` 0, ``--repeat-penalty`` 1.0, ``--seed``) and their checks
(``:555-569, 631-636``: temperature >= 0, top_p in (0, 1], max_tokens >= 1, penalty > 0).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Tuple


@dataclass(frozen=True)
class SamplingParams:
    max_tokens: int = 512            # generated tokens per request, the first one included
    temperature: float = 0.0         # 0: greedy (argmax, first index on ties)
    top_k: int = 0                   # 0: off; at most 1024 counts
    top_p: float = 1.0               # 1: off
    repeat_penalty: float = 1.0      # 1: off
    seed: Optional[int] = None       # None: taken from the clock, once per call
    stop_ids: Tuple[int, ...] = ()   # on top of the model's end-of-sequence ids
    ignore_eos: bool = False         # benchmarks: run to max_tokens
    logprobs: bool = False           # also return log p(token) of every emitted token (the reference has none)

    def __post_init__(self):
        if self.max_tokens < 1:
            raise ValueError("max_tokens must be at least 1")
        if self.temperature < 0:
            raise ValueError("temperature must be >= 0")
        if not (0.0 < self.top_p <= 1.0):
            raise ValueError("top_p must be in (0, 1]")
        if self.top_k < 0:
            raise ValueError("top_k must be >= 0")
        if self.repeat_penalty <= 0:
            raise ValueError("repeat_penalty must be > 0")


@dataclass
class GenerationResult:
    request: int                     # index of the prompt in the call
    prompt_tokens: int
    tokens: List[int] = field(default_factory=list)
    logprobs: List[float] = field(default_factory=list)      # one per token, if asked for: natural logarithm of the
                                                             # model's probability, from the logits the sampler saw
    finish_reason: str = ""          # "stop" (an end token was drawn; it is not emitted),
                                     # "length" (max_tokens), "context" (the slot is full),
                                     # "cancelled" (the call was cancelled before the request ended)
