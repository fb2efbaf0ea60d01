"""Helpers of the GPU tests: model folders from the plain implementation's random weights,
and the ways of cutting requests into steps that the tests compare."""
import json
import os
import subprocess
import sys
from typing import Dict, List, Sequence

import numpy as np
import torch

import plain_gemma3 as P

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def write_model(folder: str, cfg: dict, weights: Dict[str, torch.Tensor], dtype=torch.bfloat16) -> str:
    """config.json + model.safetensors, written with the safetensors package (not with the
    framework's own writer, so the framework's reader is checked against another writer)."""
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    save_file({k: v.to(dtype).contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    return folder


def random_tokens(n: int, vocab: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(seed)
    return [int(t) for t in torch.randint(0, vocab, (n,), generator=g)]


def plain_logits(cfg: dict, weights, tokens: Sequence[int]) -> torch.Tensor:
    return P.forward(cfg, weights, tokens, dtype=torch.float64)


# ---------------------------------------------------------------- cutting through the engine API
def run_whole(engine, tokens: Sequence[int]) -> torch.Tensor:
    slot = engine.alloc_slot()
    out = engine.step([slot], [list(tokens)], "all").float().cpu().clone()
    engine.free_slot(slot)
    return out


def run_tail(engine, tokens: Sequence[int], tail: int = 32) -> torch.Tensor:
    """First len - tail tokens in one step, the rest one by one."""
    tokens = list(tokens)
    tail = min(tail, len(tokens) - 1)
    head = tokens[:len(tokens) - tail]
    slot = engine.alloc_slot()
    parts = [engine.step([slot], [head], "all").float().cpu().clone()]
    for t in tokens[len(head):]:
        parts.append(engine.step([slot], [[t]], "all").float().cpu().clone())
    engine.free_slot(slot)
    return torch.cat(parts, 0)


def run_batched(engine, requests: Sequence[Sequence[int]], prompt_lens: Sequence[int]) -> List[torch.Tensor]:
    """One batch: the first step brings ``prompt_lens[i]`` tokens of request i, later steps one
    token each; a request leaves the batch (its slot is freed) when its tokens are used up."""
    reqs = [list(r) for r in requests]
    slots = [engine.alloc_slot() for _ in reqs]
    outs: List[List[torch.Tensor]] = [[] for _ in reqs]
    used = [min(p, len(r)) for p, r in zip(prompt_lens, reqs)]
    live = list(range(len(reqs)))
    lg = engine.step([slots[i] for i in live], [reqs[i][:used[i]] for i in live], "all").float().cpu().clone()
    off = 0
    for i in live:
        outs[i].append(lg[off:off + used[i]])
        off += used[i]
    while True:
        done = [i for i in live if used[i] >= len(reqs[i])]
        for i in done:
            engine.free_slot(slots[i])
        live = [i for i in live if used[i] < len(reqs[i])]
        if not live:
            break
        lg = engine.step([slots[i] for i in live], [[reqs[i][used[i]]] for i in live], "all").float().cpu().clone()
        for j, i in enumerate(live):
            outs[i].append(lg[j:j + 1])
            used[i] += 1
    return [torch.cat(o, 0) for o in outs]


# ---------------------------------------------------------------- bin/trace_run as a user would call it
def trace_steps_batched(batches: Sequence[Sequence[Sequence[int]]], prompt_lens: Sequence[Sequence[int]]):
    """Steps (JSON records) for batches replayed one after another; returns (records, where)
    with where[(batch, request)] = list of (step, row) for each of the request's positions."""
    records, where = [], {}
    step = 0
    for bi, (reqs, plens) in enumerate(zip(batches, prompt_lens)):
        used = [min(p, len(r)) for p, r in zip(plens, reqs)]
        live = list(range(len(reqs)))
        entries, row = [], 0
        for i in live:
            entries.append({"id": f"b{bi}r{i}", "tokens": list(reqs[i][:used[i]]), "want": list(range(used[i]))})
            where[(bi, i)] = [(step, row + k) for k in range(used[i])]
            row += used[i]
        end = [f"b{bi}r{i}" for i in live if used[i] >= len(reqs[i])]
        records.append({"step": step, "entries": entries, "end": end})
        step += 1
        live = [i for i in live if used[i] < len(reqs[i])]
        while live:
            entries = []
            for j, i in enumerate(live):
                entries.append({"id": f"b{bi}r{i}", "tokens": [reqs[i][used[i]]], "want": [0]})
                where[(bi, i)].append((step, j))
                used[i] += 1
            end = [f"b{bi}r{i}" for i in live if used[i] >= len(reqs[i])]
            records.append({"step": step, "entries": entries, "end": end})
            step += 1
            live = [i for i in live if used[i] < len(reqs[i])]
    return records, where


def run_trace_tool(model_dir: str, dtype: str, records, out_dir: str, max_tokens: int, vocab: int,
                   timeout: int = 600) -> Dict[int, np.ndarray]:
    """Run bin/trace_run as a child process; {step: logits [wanted, vocab]}."""
    os.makedirs(out_dir, exist_ok=True)
    text = "".join(json.dumps(r) + "\n" for r in records)
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir,
                           "--dtype", dtype, "--out", out_dir, "--max-tokens", str(max_tokens)],
                          input=text, capture_output=True, text=True, timeout=timeout)
    if proc.returncode != 0:
        raise RuntimeError(f"trace_run failed ({proc.returncode}):\n{proc.stderr[-4000:]}")
    done = [l for l in proc.stdout.splitlines() if l.startswith("done ")]
    assert [int(l.split()[1]) for l in done] == [r["step"] for r in records], proc.stdout[-2000:]
    out = {}
    for r in records:
        path = os.path.join(out_dir, f"{r['step']}.f32")
        if any(e.get("want") for e in r["entries"]):
            out[r["step"]] = np.fromfile(path, dtype="<f4").reshape(-1, vocab)
    return out
