"""Command line in the reference's manner: ``agave [OPTIONS] <model> [prompt]``.

Options keep the reference's names and meanings where it has them (``src/main.zig:325-382``):
``-n/--max-tokens`` (512), ``-t/--temperature`` (0 = greedy), ``--top-p`` (1.0), ``--top-k``
(0 = off), ``--repeat-penalty`` (1.0), ``--seed``, ``--ctx-size`` (0 = the model's full
context; default min(model, 4096), ``:345, 1096-1113``), ``--prefill-batch-size``, ``--json``,
``--model-info``, ``--profile``, ``-q/--quiet``, ``-V/--verbose``, ``-d/--debug``, ``-v/--version``,
``--backend`` (only ``auto`` and ``rocm`` exist here).  The reference's options for its server,
quantised caches, vision, speculative decoding, its single-dispatch kernel and grammars have no
counterpart here.  There is no tokenizer in this library: a prompt is a list
of token ids ("2 17 5" or "2,17,5"), and the output is token ids.

Added: ``--prompt-file`` (one request per line), ``--dtype``, ``--max-batch``, ``--ignore-eos``, ``--logprobs``, ``--cast-weights``,
``--random-weights CONFIG.json`` (write a random model folder at <model> first).
"""
from __future__ import annotations

import argparse
import json
import re
import sys
import time
from typing import List, Optional

def parse_ids(text: str) -> List[int]:
    parts = [p for p in re.split(r"[\s,]+", text.strip()) if p]
    try:
        return [int(p) for p in parts]
    except ValueError:
        raise SystemExit(f"error: a prompt is a list of token ids, got {text!r}") from None


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="agave_amd", description="Generate token ids with a model folder on one MI355X.")
    ap.add_argument("model", help="folder with config.json and *.safetensors")
    ap.add_argument("prompt", nargs="?", help='token ids of the prompt, e.g. "2 17 5"')
    ap.add_argument("-n", "--max-tokens", type=int, default=512, help="maximum tokens to generate [default: 512]")
    ap.add_argument("-t", "--temperature", type=float, default=0.0, help="sampling temperature, 0 = greedy [default: 0]")
    ap.add_argument("--top-p", type=float, default=1.0, help="nucleus sampling threshold [default: 1.0]")
    ap.add_argument("--top-k", type=int, default=0, help="top-k sampling, 0 = disabled [default: 0]")
    ap.add_argument("--repeat-penalty", type=float, default=1.0, help="repetition penalty [default: 1.0]")
    ap.add_argument("--seed", type=int, default=None, help="random seed for sampling [default: random]")
    ap.add_argument("--ctx-size", type=int, default=None,
                    help="context window size; 0 = full model context [default: min(model, 4096)]")
    ap.add_argument("--prefill-batch-size", type=int, default=0,
                    help="prefill chunk size in tokens; 0 = whole prompts in one step [default: 0]")
    ap.add_argument("--json", action="store_true", help="output results as JSON (implies --quiet)")
    ap.add_argument("--model-info", action="store_true", help="print model metadata and exit (supports --json)")
    ap.add_argument("--profile", action="store_true", help="profile per-op timing (lowers throughput)")
    ap.add_argument("-q", "--quiet", action="store_true", help="suppress stats (raw output only)")
    ap.add_argument("-V", "--verbose", action="store_true", help="show technical details")
    ap.add_argument("-v", "--version", action="store_true", help="print version and exit")
    ap.add_argument("-d", "--debug", action="store_true",
                    help="debug output (the token ids that are fed, per-request details); implies --verbose")
    ap.add_argument("--backend", default="auto",
                    help="compute backend: auto or rocm (the reference's other backends do not exist here) [default: auto]")
    # not in the reference
    ap.add_argument("--prompt-file", help="file with one prompt (token ids) per line; runs them as batches")
    ap.add_argument("--prompt-ids", help="token ids of the prompt (same as the positional)")
    ap.add_argument("--dtype", choices=["bfloat16", "float32", "bf16", "fp32"], default="bfloat16")
    ap.add_argument("--max-batch", type=int, default=8, help="sequences per batch [default: 8]")
    ap.add_argument("--ignore-eos", action="store_true", help="do not stop at end-of-sequence ids")
    ap.add_argument("--logprobs", action="store_true", help="with --json: the log-probability of every generated token")
    ap.add_argument("--no-bos", action="store_true", help="do not prepend the begin-of-sequence id")
    ap.add_argument("--cast-weights", action="store_true",
                    help="cast matrices that the checkpoint stores in 32-bit to the engine's dtype (default: they stay 32-bit)")
    ap.add_argument("--random-weights", metavar="CONFIG.json",
                    help="first write random weights for this configuration into <model> (uses --seed)")
    return ap


def model_info(engine) -> dict:
    s = engine.spec
    return {"architecture": s.architecture, "vocab_size": s.vocab_size, "hidden_size": s.hidden,
            "n_layers": len(s.layers), "max_context": engine.max_context, "dtype": str(engine.dtype).split(".")[-1],
            "bos_token_id": s.bos_token_id, "eos_token_ids": list(s.eos_token_ids),
            "weight_bytes": engine.model.weight_bytes(), "cache_bytes": engine.cache.bytes(),
            "cache_groups": [{"window": k.window, "n_kv_heads": k.n_kv_heads, "head_dim": k.head_dim}
                             for k in engine.cache.group_keys]}


def main(argv: Optional[List[str]] = None) -> int:
    ap = build_parser()
    if argv is None:
        argv = sys.argv[1:]
    if "-v" in argv or "--version" in argv:
        from . import __version__
        print(f"agave_amd {__version__}")
        return 0
    args = ap.parse_args(argv)
    if args.max_tokens < 1:
        ap.error("--max-tokens must be at least 1")
    if args.temperature < 0:
        ap.error("--temperature must be >= 0")
    if not (0 < args.top_p <= 1):
        ap.error("--top-p must be in (0, 1]")
    if args.repeat_penalty <= 0:
        ap.error("--repeat-penalty must be > 0")
    if args.backend not in ("auto", "rocm"):
        ap.error(f"--backend {args.backend}: this library runs on rocm (one MI355X) only")
    if args.debug:
        args.verbose = True
    quiet = args.quiet or args.json

    if args.random_weights:
        from .weights import write_random_model
        with open(args.random_weights) as f:
            write_random_model(json.load(f), args.seed or 0, args.model)

    from .engine import Engine
    from .engine.generate import GenerationStats
    from .sampling import SamplingParams

    if args.ctx_size is not None and args.ctx_size < 0:
        ap.error("--ctx-size must be >= 0")
    t0 = time.perf_counter()
    engine = Engine.from_folder(args.model, dtype=args.dtype, max_slots=max(1, args.max_batch),
                                keep_stored_precision=not args.cast_weights,
                                max_context=args.ctx_size)     # None: min(model, 4096); 0: the model's
    load_ms = (time.perf_counter() - t0) * 1e3
    if args.model_info:
        info = model_info(engine)
        print(json.dumps(info) if args.json else "\n".join(f"{k}: {v}" for k, v in info.items()))
        return 0

    prompts: List[List[int]] = []
    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompts = [parse_ids(line) for line in f if line.strip()]
    text = args.prompt_ids or args.prompt
    if text:
        prompts.append(parse_ids(text))
    bos = engine.spec.bos_token_id
    if not prompts:
        if bos is None:
            ap.error("no prompt given and the model has no begin-of-sequence id")
        prompts = [[]]                      # an empty prompt forwards the BOS alone (src/main.zig:2209-2214)
    if bos is not None and not args.no_bos:
        prompts = [p if (p and p[0] == bos) else [bos] + p for p in prompts]   # src/main.zig:2199-2208

    if args.debug and not quiet:
        for i, p in enumerate(prompts):
            print(f"[debug] request {i}: {len(p)} prompt token ids: {' '.join(map(str, p))}", file=sys.stderr)
    params = SamplingParams(max_tokens=args.max_tokens, temperature=args.temperature, top_k=args.top_k,
                            top_p=args.top_p, repeat_penalty=args.repeat_penalty, seed=args.seed,
                            ignore_eos=args.ignore_eos, logprobs=args.logprobs)
    stats = GenerationStats()
    engine.prefill_chunk = max(0, args.prefill_batch_size)
    if args.profile:
        engine.enable_profiling()
    results = engine.generate(prompts, params, stats=stats)
    table = engine.profile_table() if args.profile else None
    if table is not None and not args.json:
        whole = sum(r[2] for r in table) or 1.0
        print(f"{'op':32s} {'calls':>8s} {'ms':>10s} {'%':>6s}", file=sys.stderr)
        for name, calls, ms in table:
            print(f"{name:32s} {calls:8d} {ms:10.3f} {100 * ms / whole:6.1f}", file=sys.stderr)
    if args.json:
        extra = {"profile": [{"op": n, "calls": c, "ms": round(ms, 3)} for n, c, ms in table]} if table else {}
        print(json.dumps({**extra,
            "outputs": [{"request": r.request, "tokens": r.tokens, "finish_reason": r.finish_reason,
                         "prompt_tokens": r.prompt_tokens,
                         **({"logprobs": [round(x, 6) for x in r.logprobs]} if args.logprobs else {})} for r in results],
            "tokens": stats.tokens, "tok_per_sec": round(stats.tok_per_sec, 2),
            "prefill_tokens": stats.prefill_tokens, "prefill_ms": round(stats.prefill_ms, 3),
            "prefill_tok_per_sec": round(stats.prefill_tok_per_sec, 2), "gen_ms": round(stats.gen_ms, 3),
            "load_ms": round(load_ms, 1)}))
    else:
        for r in results:
            print(" ".join(str(t) for t in r.tokens))
        if not quiet:
            print(f"[{stats.tokens} tokens, {stats.tok_per_sec:.1f} tok/s decode | prefill {stats.prefill_tokens} tokens, "
                  f"{stats.prefill_tok_per_sec:.1f} tok/s | {stats.batches} batch(es)]", file=sys.stderr)
            if args.verbose:
                for r in results:
                    print(f"  request {r.request}: {r.prompt_tokens} prompt tokens, {len(r.tokens)} generated, "
                          f"finish={r.finish_reason}", file=sys.stderr)
    return 0
