"""The engine: a model on one GPU with its cache, its step function and generation.

Programmatic surface in the manner of the reference's ``Model`` interface
(``src/models/model.zig:205-307``: ``forward``, ``prefill``, ``getLogits``, ``resetCache``,
``eosId``, ``vocabSize``, ``nLayers``, ``kvSeqLen``), for a batch of sequences in slots:

    engine = Engine.from_folder(model_dir, dtype="bfloat16", max_slots=8, max_context=4096)
    slot = engine.alloc_slot()
    logits = engine.step([slot], [[2, 17, 5]], want="last")      # float32 [1, vocab] on the GPU
    engine.free_slot(slot)
    results = engine.generate(prompts, SamplingParams(temperature=0.8, seed=1))
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import os
import threading

import torch

from ..cache import PAGE, GroupKey, KVCache, pool_pages
from ..config import find_architecture, read_config_json
from ..config.spec import ModelSpec
from ..parts import BuildEnv, Workspace
from ..weights import Checkpoint, DictWeightSource, RandomWeightSource, WeightSource
from .graphs import PROMPT_GRAPH_PAD, PROMPT_GRAPH_TOKENS, DecodeGraphs, span_bucket
from .model import Model, tensor_needs
from .step import Step, StepPlanner, Want, resolve_want, split_pieces

DEFAULT_CONTEXT = 4096      # the reference's default context (src/main.zig:107, 1100-1113)
DEFAULT_PIECE = 4096        # tokens a sequence brings at most in one run of the model

_DTYPES = {"float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
           "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
           torch.float32: torch.float32, torch.bfloat16: torch.bfloat16}


def parse_dtype(dtype) -> torch.dtype:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError(f"dtype must be bfloat16 or float32, got {dtype!r}") from None


def require_gpu(device=None) -> torch.device:
    """The MI355X the engine runs on.  There is no CPU path."""
    if not torch.cuda.is_available():
        raise RuntimeError("agave_amd needs a GPU: no HIP device is visible (there is no CPU fallback)")
    dev = torch.device(device if device is not None else "cuda:0")
    if dev.type != "cuda":
        raise RuntimeError(f"agave_amd runs on the GPU only, got device {dev}")
    return dev


class Engine:
    def __init__(self, spec: ModelSpec, weights, *, dtype="bfloat16", max_slots: int = 8,
                 max_context: Optional[int] = None, cache_tokens: Optional[int] = None,
                 prefill_piece: Optional[int] = None, keep_stored_precision: bool = True, device=None,
                 config=None, will_sample: bool = True):
        """``max_context``: longest sequence a slot may hold; None: the smaller of the model's
        context and 4096, 0: the model's whole context (the reference's ``--ctx-size``,
        ``src/main.zig:1100-1113``, ``src/models/gemma3.zig:164-166``).
        ``cache_tokens``: positions the cache holds over all live sequences, each counted
        rounded up to a multiple of 64 (default: ``max_slots * max_context``).
        ``prefill_piece``: most tokens of one sequence that the model runs at a time (default
        4096); a longer prompt enters in pieces.  Layers with a window keep only the window's
        reach plus one piece per sequence, so their share of the cache does not grow with
        the context.
        ``keep_stored_precision``: in a bfloat16 engine a matrix that the checkpoint stores in
        32-bit stays in 32-bit (its products then run on the plain multiply-add kernel, far from
        the matrix cores' speed; a line on standard error says how many do); False casts such
        matrices to bfloat16 at load.  Half precision is always cast to the engine's type.
        ``will_sample`` False: the sampling kernels are not built with the others at construction (a
        caller that only reads logits never needs them; they would still be built at first use)."""
        self.device = require_gpu(device)
        self.dtype = parse_dtype(dtype)
        self._cancel = threading.Event()
        self.spec = spec
        self.config = config
        torch.cuda.set_device(self.device)
        # what this element type needs is compiled now, side by side, rather than one library
        # after the other as the first step meets them (a fresh checkout's first run)
        from ..ops import library
        needed = ["elementwise", "gemm", "attention_plain"]
        if will_sample:                    # (a caller that only wants logits, like trace replay, builds no sampling kernels)
            needed.append("sampling")
        if self.dtype == torch.bfloat16:
            needed += ["gemm_mfma", "attention_mfma"]
        library.ensure_built(needed)
        self.workspace = Workspace(self.device)
        self.env = BuildEnv(self.dtype, self.device, self.workspace, keep_stored_precision=bool(keep_stored_precision))
        self.model = Model(spec, weights, self.env)
        if self.env.kept_32bit:
            kept = self.env.kept_32bit
            library._log(f"{len(kept)} weight matrices are stored in 32-bit and stay so ({', '.join(sorted(set(kept)))}): "
                         f"their products run on the plain multiply-add kernel, not on the matrix cores; "
                         f"keep_stored_precision=False (--cast-weights) casts them to bfloat16")
        if max_context is None:
            self.max_context = min(int(spec.max_context), DEFAULT_CONTEXT)
        else:
            self.max_context = int(max_context) if int(max_context) > 0 else int(spec.max_context)
        if self.max_context < 1:
            raise ValueError("max_context must be positive")
        self.max_piece = min(self.max_context, int(prefill_piece) if prefill_piece else DEFAULT_PIECE)
        if self.max_piece < 1:
            raise ValueError("prefill_piece must be positive")
        kv_needs = self.model.kv_needs()
        pages: Dict[GroupKey, int] = {}
        for key in set(kv_needs.values()):
            # what max_slots sequences can hold at most; fewer if the caller bounds the live positions
            pages[key] = pool_pages(key.window, max_slots, self.max_context, self.max_piece)
            if cache_tokens is not None:
                pages[key] = min(pages[key], max(1, (int(cache_tokens) + PAGE - 1) // PAGE))
        self.cache = KVCache(kv_needs, self.model.state_needs(), max_slots, pages, self.dtype, self.device,
                             self.max_context)
        self.planner = StepPlanner(self.cache, spec.vocab_size, self.device, self.workspace)
        self.prefill_chunk = 0          # > 0: prompts enter in pieces of at most this many tokens (at most max_piece)
        self.use_graphs = os.environ.get("AGAVE_AMD_NO_GRAPHS", "") not in ("1", "true", "yes")
        self.graphs = DecodeGraphs(self)
        # prompts are recorded only if every mixer and feed-forward says that its multi-token steps can be
        # (no host-side work that depends on the tokens, nothing that waits for the GPU)
        self._prompt_graphs_ok = all(getattr(b.mixer, "prompt_steps_can_be_recorded", False) and
                                     (b.ffn is None or getattr(b.ffn, "prompt_steps_can_be_recorded", False))
                                     for b in self.model.blocks)
        self._decode_widths = [g.table_width(self.max_context, 1) for g in self.cache.groups]

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_folder(cls, model_dir: str, **kw) -> "Engine":
        """A folder with config.json and safetensors; the model class is chosen by config.json."""
        raw = read_config_json(model_dir)
        arch = find_architecture(raw)
        cfg = arch.parse(raw)
        ckpt = Checkpoint(model_dir)
        spec = arch.spec(cfg, ckpt.names())
        weights = WeightSource(ckpt, tensor_needs(spec), spec.tensor_scope)
        return cls(spec, weights, config=cfg, **kw)

    @classmethod
    def from_tensors(cls, raw_config: dict, tensors: Dict[str, torch.Tensor], **kw) -> "Engine":
        arch = find_architecture(raw_config)
        cfg = arch.parse(raw_config)
        spec = arch.spec(cfg, tensors.keys())
        return cls(spec, DictWeightSource(tensors, tensor_needs(spec), scope=spec.tensor_scope), config=cfg, **kw)

    @classmethod
    def from_random(cls, raw_config: dict, seed: int = 0, **kw) -> "Engine":
        """Random weights made on the GPU (for measurements; no folder is written)."""
        arch = find_architecture(raw_config)
        cfg = arch.parse(raw_config)
        spec = arch.spec(cfg, None)
        device = require_gpu(kw.get("device"))
        wdtype = parse_dtype(kw.get("dtype", "bfloat16"))
        return cls(spec, RandomWeightSource(tensor_needs(spec), seed, device, wdtype), config=cfg, **kw)

    # ------------------------------------------------------------------ the reference's accessors
    @property
    def vocab_size(self) -> int:
        return self.spec.vocab_size

    @property
    def n_layers(self) -> int:
        return len(self.spec.layers)

    @property
    def eos_ids(self):
        return tuple(self.spec.eos_token_ids)

    def kv_seq_len(self, slot: int) -> int:
        return self.cache.length(slot)

    def enable_profiling(self, on: bool = True) -> None:
        """Time every kernel call by class (``profile_table``).  Steps run eagerly meanwhile, with
        two events around each call, so throughput drops (the reference's ``--profile``,
        ``src/main.zig:381, 1516``)."""
        from ..ops import library
        library.profile.enabled = bool(on)
        library.profile.reset()
        self._graphs_before_profiling = getattr(self, "_graphs_before_profiling", self.use_graphs)
        self.use_graphs = False if on else self._graphs_before_profiling

    def profile_table(self):
        """(op, calls, total ms) rows by falling time."""
        from ..ops import library
        return library.profile.table()

    # ------------------------------------------------------------------ slots and steps
    def alloc_slot(self) -> int:
        return self.cache.alloc_slot()

    def free_slot(self, slot: int) -> None:
        self.cache.free_slot(slot)

    def step(self, slots: Sequence[int], tokens: Sequence[Sequence[int]], want: Want = "last") -> Optional[torch.Tensor]:
        """Run ``tokens[i]`` as the next tokens of the sequence in ``slots[i]``.  Returns the
        float32 logits [wanted, vocab] on the GPU in the order of the sequences and of their
        wanted places (valid until the next step), or None if nothing is wanted."""
        return self._run(slots, tokens, want)[0]

    def _run(self, slots, tokens, want, carry=None, floats=None):
        """Run one step of the caller's; (logits, the last planned step).  A step in which a
        sequence brings more tokens than a piece holds runs as several steps of the model, the
        last of which holds every sequence; the logits come back in the caller's order."""
        piece = min(self.max_piece, int(self.prefill_chunk)) if int(self.prefill_chunk or 0) > 0 else self.max_piece
        n_new = [len(t) for t in tokens]
        if n_new and max(n_new) > piece and len(slots) == len(tokens) and min(n_new) >= 1:
            return self._run_in_pieces(slots, tokens, want, piece, floats)
        return self._run_one(slots, tokens, want, carry, floats)

    def _run_in_pieces(self, slots, tokens, want, piece, floats):
        n_new = [len(t) for t in tokens]
        wanted = resolve_want(want, n_new)
        pieces = split_pieces(n_new, piece)
        self.cache.check_pieces(list(slots), pieces)       # all or nothing, before the first piece runs
        # where every wanted row of the caller's order comes from: (piece, row among that piece's wanted rows)
        first_row = [0]
        for w in wanted:
            first_row.append(first_row[-1] + len(w))
        total = first_row[-1]
        done = [0] * len(slots)
        result = None
        gathered = None
        for j, counts in enumerate(pieces):
            idx = [i for i, c in enumerate(counts) if c > 0]
            sub_tokens = [tokens[i][done[i]:done[i] + counts[i]] for i in idx]
            sub_want, dest = [], []
            for i in idx:
                lo, hi = done[i], done[i] + counts[i]
                places = [(k, x - lo) for k, x in enumerate(wanted[i]) if lo <= x < hi]
                sub_want.append([x for _, x in places])
                dest += [first_row[i] + k for k, _ in places]
            last = j == len(pieces) - 1
            logits, step = self._run_one([slots[i] for i in idx], sub_tokens, sub_want, None, floats if last else None)
            for i in idx:
                done[i] += counts[i]
            if logits is None:
                continue
            if last and len(dest) == total:
                result = logits                             # everything wanted lies in the last piece, in order
            else:
                if gathered is None:
                    gathered = self.workspace.get("logits_gathered", total, self.spec.vocab_size, torch.float32)
                gathered.index_copy_(0, torch.tensor(dest, dtype=torch.int64, device=self.device), logits)
                result = gathered
        return (result if total else None), step

    def _run_one(self, slots, tokens, want, carry=None, floats=None):
        """Plan, run and commit one step of the model; (logits, step)."""
        # a short prompt of one sequence that wants its last row: padded to a few rows' multiple, so that it
        # can be replayed as a graph (the host needs longer to launch such a step than the GPU to run it)
        as_prompt_graph = (self.use_graphs and self._prompt_graphs_ok and carry is None and len(slots) == 1
                           and len(tokens) == 1 and 2 <= len(tokens[0]) <= PROMPT_GRAPH_TOKENS
                           and isinstance(want, str) and want == "last")
        step = self.planner.plan(slots, tokens, want, decode_widths=self._decode_widths if self.use_graphs else None,
                                 carry=carry, floats=floats, pad_to=PROMPT_GRAPH_PAD if as_prompt_graph else 0)
        if carry is not None:
            from ..ops import sampling as sample_ops
            sample_ops.gather_tokens(self._sampled_all(), step.carry_dev, step.tokens)
        if self.use_graphs and step.is_decode and step.n_want == step.n_tokens:
            step.fixed_span = span_bucket(step.page_span(None))
            logits = self.graphs.run(step)
        elif as_prompt_graph and step.n_tokens <= PROMPT_GRAPH_TOKENS:
            logits = self.graphs.run_prompt(step)
        else:
            logits = self.model.forward(step)
        self.planner.commit(step)
        return logits, step

    # ------------------------------------------------------------------ cancelling from another thread
    def cancel(self) -> None:
        """Ask the running :meth:`generate` call to stop after the step that is under way (the
        reference's ``cancel``, ``src/models/model.zig:238-241``).  Safe to call from any thread."""
        self._cancel.set()

    def cancel_requested(self) -> bool:
        return self._cancel.is_set()

    def clear_cancel(self) -> None:
        self._cancel.clear()

    def synchronize(self) -> None:
        torch.cuda.synchronize(self.device)

    # ------------------------------------------------------------------ sampling and generation
    @property
    def max_slots(self) -> int:
        return self.cache.max_slots

    def _sampled_all(self) -> torch.Tensor:
        """Where every step leaves its sampled tokens (one per sequence, in the step's order)."""
        return self.workspace.get("sampled", self.max_slots, 1, torch.int32).view(-1)

    def step_sample(self, slots: Sequence[int], tokens: Sequence[Sequence[int]], rows) -> List[int]:
        """One step, then one token per sequence drawn from its last logits on the GPU.
        ``rows``: one :class:`RowSampling` per sequence."""
        return self.finish_step(self.launch_step(slots, tokens, rows))

    def launch_step(self, slots: Sequence[int], tokens: Optional[Sequence[Sequence[int]]], rows,
                    carry: Optional[Sequence[int]] = None):
        """Enqueue a step and the sampling of one token per sequence, without waiting for the
        GPU; :meth:`finish_step` returns the tokens.  ``carry`` (with ``tokens`` None): sequence i
        of this step continues with the token that row ``carry[i]`` of the step launched before
        sampled; it is taken on the device, so this step can be launched before that one has
        been read back, and the host's work on a step hides behind the GPU's on the one before."""
        import numpy as np
        from ..ops import sampling as sample_ops
        b = len(slots)
        if carry is not None:
            if tokens is not None:
                raise ValueError("launch_step: either tokens or carry")
            if any(r.repeat_penalty != 1.0 for r in rows):
                raise ValueError("launch_step: the repeat penalty needs the tokens on the host; no carry")
            tokens = [[0]] * b
        params = np.asarray([[r.temperature, float(min(r.top_k, 1 << 20)), r.top_p, r.u] for r in rows],
                            dtype=np.float32)
        logits, step = self._run(slots, tokens, "last", carry=carry, floats=params)
        if any(r.repeat_penalty != 1.0 and r.generated for r in rows):
            cu = [0]
            flat: List[int] = []
            for r in rows:
                if r.repeat_penalty != 1.0:
                    flat.extend(r.generated)
                cu.append(len(flat))
            ids = torch.tensor(flat or [0], dtype=torch.int32, device=self.device)
            cu_t = torch.tensor(cu, dtype=torch.int32, device=self.device)
            pen = torch.tensor([r.repeat_penalty for r in rows], dtype=torch.float32, device=self.device)
            sample_ops.repeat_penalty(logits, ids, cu_t, pen)
        work = self.workspace.get("sample_work", b, self.spec.vocab_size, torch.float32)
        out = self._sampled_all()[:b]
        scratch = self.workspace.get("sample_scratch", b, sample_ops.scratch_words(), torch.float32).view(-1)
        sample_ops.sample(logits, work, step.floats_dev.view(b, 4), out, scratch,
                          kinds=sample_ops.kinds_of(rows, self.spec.vocab_size))
        # the host gets the tokens, and behind them the drawn tokens' log-probabilities (as bits) if any row wants them
        want_lp = any(getattr(r, "logprob", False) for r in rows)
        lp_dev = None
        if want_lp:
            lp_dev = self.workspace.get("sampled_logprob", self.max_slots, 1, torch.float32).view(-1)[:b]
            sample_ops.token_logprob(logits, out, lp_dev)
        self._result_turn = 1 - getattr(self, "_result_turn", 0)
        hosts = getattr(self, "_result_hosts", None)
        if hosts is None:
            hosts = self._result_hosts = [torch.empty(2 * self.max_slots, dtype=torch.int32, pin_memory=True)
                                          for _ in range(2)]
        host = hosts[self._result_turn]
        host[:b].copy_(out, non_blocking=True)
        if want_lp:
            host[self.max_slots:self.max_slots + b].copy_(lp_dev.view(torch.int32), non_blocking=True)
        done = torch.cuda.Event()
        done.record()
        return host, done, b, want_lp

    def finish_step(self, handle) -> List[int]:
        """The tokens of a step that :meth:`launch_step` enqueued (waits for it)."""
        host, done, b, want_lp = handle
        done.synchronize()
        # (what generation reads after every step: the step's log-probabilities, or None)
        self.last_logprobs = host[self.max_slots:self.max_slots + b].view(torch.float32).tolist() if want_lp else None
        return host[:b].tolist()

    def generate(self, prompts, params=None, max_batch: Optional[int] = None, stats=None):
        """Generate for every prompt (lists of token ids); see :func:`agave_amd.engine.generate.generate`."""
        from ..sampling import SamplingParams
        from .generate import generate
        return generate(self, prompts, params if params is not None else SamplingParams(),
                        eos_ids=self.spec.eos_token_ids, max_batch=max_batch, stats=stats)
