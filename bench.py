"""Decode and prefill throughput of the Gemma 3 4B text decoder (random bf16 weights) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one decode step of the whole batch: planning on the host, every kernel of the
model, sampling (greedy) and the copy of the new token ids back to the host; as in generation,
a step is launched while the host still waits for the tokens of the step before.  The default run
has the layer sizes of the published Gemma 3 4B text configuration, a batch of 8, prompts of 1,024 tokens and
256 decoded tokens per sequence (W warm-up steps, then K timed ones).  One JSON line is
printed: ``value`` is decoded tokens a second; ``prefill`` is one 2,048-token prompt;
``roofline`` prices the decode step by the bytes it has to read (every weight once, and the
cache of the live requests) against 8 TB/s; ``points`` holds decode at batch 1 and 64 and
prompts of 256 and 512 tokens (tokens a second each);
``peaks_measured`` is what this machine delivered to a streaming read and to a loop of
matrix-core instructions on random data a moment before (the fractions stay against the
published peaks).

The other published shapes:

    python bench.py --model 12b --ragged 16 --context 8192        # 16 prompts of unequal lengths 64..4096
    python bench.py --model 27b --prompt-len 2048 --context 8192 --batch 1 --no-points
    python bench.py --model 27b --prompt-len 2048 --context 8192 --batch 32 --no-points
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0            # MI355X HBM3E, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

# Gemma 3 4B text decoder, as its config.json gives it
GEMMA3_4B = dict(
    architectures=["Gemma3ForCausalLM"], model_type="gemma3_text", vocab_size=262208, hidden_size=2560,
    num_hidden_layers=34, num_attention_heads=8, num_key_value_heads=4, head_dim=256,
    query_pre_attn_scalar=256, intermediate_size=10240, sliding_window=1024, sliding_window_pattern=6,
    rope_theta=1e6, rope_local_base_freq=1e4, rope_scaling={"rope_type": "linear", "factor": 8.0},
    rms_norm_eps=1e-6, tie_word_embeddings=True, hidden_activation="gelu_pytorch_tanh",
    max_position_embeddings=131072, bos_token_id=2, eos_token_id=1)

# the larger published sizes of the same architecture, for --model (not the default run)
GEMMA3_12B = dict(GEMMA3_4B, hidden_size=3840, num_hidden_layers=48, num_attention_heads=16, num_key_value_heads=8,
                  intermediate_size=15360)
GEMMA3_27B = dict(GEMMA3_4B, hidden_size=5376, num_hidden_layers=62, num_attention_heads=32, num_key_value_heads=16,
                  head_dim=128, query_pre_attn_scalar=168, intermediate_size=21504)
MODELS = {"4b": ("gemma3-4b-text", GEMMA3_4B), "12b": ("gemma3-12b-text", GEMMA3_12B),
          "27b": ("gemma3-27b-text", GEMMA3_27B)}

PROMPT_LEN, DECODE_LEN, CONTEXT, PREFILL_LEN = 1024, 256, 4096, 2048


def model_numbers(cfg: dict, n_layers: int):
    e, nh, nkv, hd = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    ff, v = cfg["intermediate_size"], cfg["vocab_size"]
    qd, kvd = nh * hd, nkv * hd
    pattern = cfg["sliding_window_pattern"]
    sliding = [(i + 1) % pattern != 0 for i in range(n_layers)]
    per_layer = e * (qd + 2 * kvd) + qd * e + 3 * e * ff
    norms = n_layers * (4 * e + 2 * hd) + e
    return dict(e=e, qd=qd, kvd=kvd, ff=ff, v=v, sliding=sliding, window=cfg["sliding_window"],
                linear_params=per_layer * n_layers, table_params=v * e, norm_params=norms)


def decode_step_bytes(m: dict, contexts) -> float:
    """Bytes one decode step has to read: every weight once (bf16; the tied table once, as the
    output matrix; norm gains in 32-bit) and the keys and values each live request attends to."""
    weights = 2 * (m["linear_params"] + m["table_params"]) + 4 * m["norm_params"]
    kv = 0
    for ctx in contexts:
        for s in m["sliding"]:
            kv += (min(ctx, m["window"]) if s else ctx) * m["kvd"] * 2 * 2
    return float(weights + kv)


def measured_peaks():
    """What the machine delivers just now: a streaming read of 2 GiB and a loop of bfloat16
    matrix-core instructions on normally distributed operands (the published peak holds for zeros)."""
    from agave_amd.ops import peaks
    return {"hbm_read_gbs": round(peaks.hbm_read_gbs(), 1), "mfma_bf16_tflops": round(peaks.mfma_bf16_tflops(), 1)}


def prefill_flops(m: dict, t: int) -> float:
    """Multiply-adds of one prompt of t tokens, twice: the linear layers on every token, the
    output matrix on the one wanted row, and attention over the visible pairs."""
    linear = 2.0 * t * m["linear_params"] + 2.0 * m["table_params"]
    attn = 0.0
    for s in m["sliding"]:
        pairs = sum(min(i + 1, m["window"]) for i in range(t)) if s else t * (t + 1) // 2
        attn += 4.0 * m["qd"] * pairs
    return linear + attn


def random_prompts(n: int, length: int, vocab: int, seed: int):
    import numpy as np
    rng = np.random.default_rng(seed)
    return [rng.integers(0, vocab, size=length).tolist() for _ in range(n)]


def ragged_lengths(n: int, lo: int, hi: int, seed: int):
    """n prompt lengths drawn uniformly from lo..hi, the two ends among them."""
    import numpy as np
    rng = np.random.default_rng(seed)
    lens = rng.integers(lo, hi + 1, size=n).tolist()
    if n >= 2:
        lens[0], lens[-1] = lo, hi
    return lens


def run_decode(engine, batch: int, steps: int, warmup: int, seed: int, prompt_len: int = PROMPT_LEN, lengths=None,
               first_step=None):
    """Prefill ``batch`` prompts of ``prompt_len`` tokens (or of the given unequal ``lengths``, then
    as one ragged step whose time goes into ``first_step``), then time ``steps`` decode steps."""
    import numpy as np
    import torch
    from agave_amd.engine.generate import RowSampling
    if lengths is None:
        prompts = random_prompts(batch, prompt_len, engine.vocab_size, seed)
    else:
        rng = np.random.default_rng(seed)
        prompts = [rng.integers(0, engine.vocab_size, size=n).tolist() for n in lengths]
    plens = [len(p) for p in prompts]
    slots = [engine.alloc_slot() for _ in range(batch)]
    rows = [RowSampling(0.0, 0, 1.0, 1.0, 0.0, []) for _ in range(batch)]
    try:
        engine.prefill_chunk = 2048 if (batch > 8 and lengths is None) else 0
        if lengths is not None:             # the unequal prompts in one step, as a batch starts
            engine.step_sample(slots, prompts, rows)            # once untimed: libraries, workspace
            for s in slots:
                engine.free_slot(s)
            slots[:] = [engine.alloc_slot() for _ in range(batch)]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            toks = engine.step_sample(slots, prompts, rows)
            torch.cuda.synchronize()
            if first_step is not None:
                first_step.update(tokens=sum(plens), ms=round((time.perf_counter() - t0) * 1e3, 3))
        elif batch > 8:                     # keep the untimed prefill's workspace small
            toks = None
            for i in range(0, batch, 8):
                part = engine.step_sample(slots[i:i + 8], prompts[i:i + 8], rows[i:i + 8])
                toks = part if toks is None else toks + part
        else:
            toks = engine.step_sample(slots, prompts, rows)
        for _ in range(warmup):
            toks = engine.step_sample(slots, [[t] for t in toks], rows)
        torch.cuda.synchronize()
        # the timed steps run as generation runs them: each is launched, its tokens taken on the
        # device from the step before, while the host still waits for that step's tokens
        carry = list(range(batch))
        t0 = time.perf_counter()
        running = engine.launch_step(slots, [[t] for t in toks], rows)
        for _ in range(steps - 1):
            following = engine.launch_step(slots, None, rows, carry)
            toks = engine.finish_step(running)
            running = following
        toks = engine.finish_step(running)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        # keys the first timed step attends to: the prompt, the warm-up steps' tokens and its own
        contexts = [n + warmup + 1 + (steps - 1) / 2.0 for n in plens]
        return dt, contexts
    finally:
        for s in slots:
            engine.free_slot(s)
        engine.prefill_chunk = 0


def run_prefill(engine, seed: int, repeats: int = 3, length: int = PREFILL_LEN):
    import torch
    from agave_amd.engine.generate import RowSampling
    prompt = random_prompts(1, length, engine.vocab_size, seed)
    row = [RowSampling(0.0, 0, 1.0, 1.0, 0.0, [])]
    times = []
    for r in range(repeats + 1):                     # the first pass warms up
        slot = engine.alloc_slot()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step_sample([slot], prompt, row)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        engine.free_slot(slot)
        if r > 0:
            times.append(dt)
    return min(times)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=240)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--model", default="4b", choices=sorted(MODELS),
                    help="layer sizes: Gemma 3 4B (the default run), 12B or 27B")
    ap.add_argument("--layers", type=int, default=0,
                    help="run fewer layers of the same sizes (reported in config)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--prompt-len", type=int, default=PROMPT_LEN,
                    help="tokens of every prompt before the decode steps (the default run: 1024)")
    ap.add_argument("--context", type=int, default=CONTEXT, help="longest sequence a slot may hold")
    ap.add_argument("--prefill-len", type=int, default=PREFILL_LEN, help="tokens of the prefill prompt (the default run: 2048)")
    ap.add_argument("--ragged", type=int, default=0, metavar="N",
                    help="N prompts of unequal lengths 64..4096 (seeded) as one first step, then decode steps; "
                         "replaces --batch and --prompt-len")
    ap.add_argument("--no-points", action="store_true", help="skip prefill and the batch 1 / 64 points")
    ap.add_argument("--prefill-only", action="store_true",
                    help="time only the 2048-token prefill and print its record (for profiles)")
    args = ap.parse_args()
    world = int(os.environ.get("WORLD_SIZE", "1"))
    if args.gpus != 1 or world != 1:
        if int(os.environ.get("RANK", "0")) == 0:
            print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    lengths = None
    if args.ragged:
        lengths = ragged_lengths(args.ragged, 64, min(4096, args.context // 2), seed=7)
        args.batch, args.prompt_len, args.no_points = args.ragged, max(lengths), True
    if args.steps + args.warmup > args.context - args.prompt_len:
        ap.error(f"--steps + --warmup must stay within {args.context - args.prompt_len} decoded tokens")

    import torch
    from agave_amd.engine import Engine

    model_name, full = MODELS[args.model]
    if args.layers <= 0:
        args.layers = full["num_hidden_layers"]
    cfg = dict(full, num_hidden_layers=args.layers)
    m = model_numbers(cfg, args.layers)
    max_batch = args.batch if args.no_points else max(args.batch, 64)
    per_seq = -(-(args.prompt_len + max(DECODE_LEN, args.steps + args.warmup) + 64) // 64) * 64
    cache_tokens = max(max_batch * per_seq, -(-max(PREFILL_LEN, args.prefill_len) // 64) * 64 + 64)
    peaks = measured_peaks() if args.dtype == "bfloat16" else None
    engine = Engine.from_random(cfg, seed=0, dtype=args.dtype, max_slots=max_batch, max_context=args.context,
                                cache_tokens=cache_tokens, device="cuda:0")
    dkey = "bf16" if args.dtype == "bfloat16" else "fp32"
    if args.prefill_only:
        pdt = run_prefill(engine, seed=2, length=args.prefill_len)
        print(json.dumps({"prefill": {"value": round(args.prefill_len / pdt, 1), "tokens": args.prefill_len,
                                      "ms": round(pdt * 1e3, 3),
                                      "frac": round(prefill_flops(m, args.prefill_len) / pdt / PEAK_FLOPS[dkey], 4)}}),
              flush=True)
        return 0

    first_step = {}
    dt, contexts = run_decode(engine, args.batch, args.steps, args.warmup, seed=1, prompt_len=args.prompt_len,
                              lengths=lengths, first_step=first_step)
    ms_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    need = decode_step_bytes(m, contexts)
    achieved = need / (ms_step * 1e-3) / 1e9
    out = {
        "metric": f"decode tok/s, Gemma3-{args.model.upper()} {dkey}, batch {args.batch}, "
                  + (f"prompts of unequal lengths {min(lengths)}..{max(lengths)}" if lengths else f"{args.prompt_len}-token prompts")
                  + f" + {args.warmup + args.steps + 1} decoded ({args.steps} steps timed after {args.warmup} of warm-up)",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dkey, "data": "synthetic: uniform-random token ids, random N(0,0.02) weights",
        "config": {"model": model_name, "layers": args.layers, "layers_of_config": full["num_hidden_layers"],
                   "hidden": m["e"], "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
                   "head_dim": cfg["head_dim"], "intermediate": m["ff"], "vocab": m["v"],
                   "sliding_window": m["window"], "sliding_pattern": cfg["sliding_window_pattern"],
                   "global_batch": args.batch, "seq_len": args.prompt_len + args.warmup + args.steps + 1,
                   "prompt_len": args.prompt_len,
                   "context": args.context, "prefill_len": args.prefill_len, "parallelism": "single GPU",
                   "sampling": "greedy", "weights_gb": round(2 * (m["linear_params"] + m["table_params"]) / 1e9, 3)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if peaks is not None:
        out["peaks_measured"] = peaks
    if lengths:
        flops = sum(prefill_flops(m, n) for n in lengths)
        out["ragged_prefill"] = {"value": round(first_step["tokens"] / (first_step["ms"] * 1e-3), 1),
                                 "tokens": first_step["tokens"], "ms": first_step["ms"], "sequences": len(lengths),
                                 "frac": round(flops / (first_step["ms"] * 1e-3) / PEAK_FLOPS[dkey], 4)}
    if not args.no_points:
        pdt = run_prefill(engine, seed=2, length=args.prefill_len)
        flops = prefill_flops(m, args.prefill_len)
        out["prefill"] = {"value": round(args.prefill_len / pdt, 1), "tokens": args.prefill_len, "ms": round(pdt * 1e3, 3),
                          "frac": round(flops / pdt / PEAK_FLOPS[dkey], 4)}
        points = {}
        for b, k in ((1, 64), (64, 32)):
            d, _ = run_decode(engine, b, k, 8, seed=3 + b)
            points[f"decode_b{b}"] = round(b * k / d, 2)
        for n in (256, 512):                      # short prompts: tokens a second of one prompt of n tokens
            points[f"prefill_{n}"] = round(n / run_prefill(engine, seed=5, length=n), 1)
        out["points"] = points
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
