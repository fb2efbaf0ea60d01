"""Generation, the command line and the replay tool on the GPU, against the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import engine_utils as U
import plain_gemma3 as P

pytestmark = pytest.mark.gpu
ROOT = U.ROOT


@pytest.fixture(scope="module")
def model_a(tmp_path_factory):
    cfg = P.tiny_config("A")
    w = P.random_weights(cfg, 0)
    return cfg, w, U.write_model(str(tmp_path_factory.mktemp("genA")), cfg, w)


@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    cfg = P.tiny_config("B")
    w = P.random_weights(cfg, 1)
    return cfg, w, U.write_model(str(tmp_path_factory.mktemp("genB")), cfg, w)


def plain_greedy(cfg, w, prompt, n, stops=()):
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = P.argmax_first(P.forward(cfg, w, toks)[-1])
        if nxt in stops:
            break
        out.append(nxt)
        toks.append(nxt)
    return out


def test_greedy_generation_through_the_entry_point(model_a):
    """The Tiny A run: prompts of 5 / 19 / 40 tokens, 8 greedy steps each, context 64."""
    from agave_amd import Engine, SamplingParams
    cfg, w, folder = model_a
    eng = Engine.from_folder(folder, dtype="float32", max_slots=3, max_context=64)
    prompts = [U.random_tokens(n, 512, 80 + i) for i, n in enumerate((5, 19, 40))]
    res = eng.generate(prompts, SamplingParams(max_tokens=8, ignore_eos=True))
    for r, p in zip(res, prompts):
        assert r.tokens == plain_greedy(cfg, w, p, 8), f"request {r.request}"
        assert r.finish_reason == "length"
    # the same one request at a time, and with prompts entering in chunks of 7 tokens
    eng.prefill_chunk = 7
    alone = [eng.generate([p], SamplingParams(max_tokens=8, ignore_eos=True))[0].tokens for p in prompts]
    assert alone == [r.tokens for r in res]
    assert eng.cache.slots.n_free == 3


def test_stop_ids_and_context_end_generation(model_a):
    from agave_amd import Engine, SamplingParams
    cfg, w, folder = model_a
    eng = Engine.from_folder(folder, dtype="float32", max_slots=2, max_context=64)
    prompt = U.random_tokens(9, 512, 90)
    free = plain_greedy(cfg, w, prompt, 6)
    stop = free[3]
    res = eng.generate([prompt], SamplingParams(max_tokens=6, stop_ids=(stop,)))[0]
    assert res.tokens == free[:free.index(stop)] and res.finish_reason == "stop"
    long = U.random_tokens(60, 512, 91)
    res = eng.generate([long], SamplingParams(max_tokens=50, ignore_eos=True))[0]
    assert res.finish_reason == "context" and len(res.tokens) == 5       # 60 + 4 fed tokens fill the 64 positions
    assert res.tokens == plain_greedy(cfg, w, long, 5)


def test_temperature_sampling_is_seeded_and_independent_of_batch_mates(model_b):
    """The Tiny B run: prompts of 1 / 7 / 13 / 30 / 57 tokens, 12 steps at temperature 0.8."""
    from agave_amd import Engine, SamplingParams
    cfg, w, folder = model_b
    eng = Engine.from_folder(folder, dtype="float32", max_slots=5, max_context=96)
    prompts = [U.random_tokens(n, 1000, 100 + i) for i, n in enumerate((1, 7, 13, 30, 57))]
    sp = SamplingParams(max_tokens=12, temperature=0.8, seed=1, ignore_eos=True)
    a = [r.tokens for r in eng.generate(prompts, sp)]
    b = [r.tokens for r in eng.generate(prompts, sp)]
    assert a == b and all(len(t) == 12 for t in a)
    c = [r.tokens for r in eng.generate(prompts, sp, max_batch=2)]       # other batch mates, other slots
    assert c == a
    d = [r.tokens for r in eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.8, seed=2, ignore_eos=True))]
    assert d != a
    # every drawn token follows the plain rule for the u of the request's own stream
    rng = np.random.default_rng([1, 3])
    toks = list(prompts[3])
    for got in a[3]:
        u = float(rng.random(dtype=np.float32))
        want = P.sample_token(P.forward(cfg, w, toks)[-1].float(), 0.8, 0, 1.0, u)
        assert got == want
        toks.append(got)


def test_sampling_kinds_mixed_in_a_batch_with_a_large_vocabulary(tmp_path):
    """A vocabulary of 5,003 takes the sampler that shares a row among workgroups: greedy,
    temperature, top-k and top-p requests in one batch, each following the plain rule for the u
    of its own stream."""
    from agave_amd import Engine, SamplingParams
    cfg = dict(P.tiny_config("A"), vocab_size=5003)
    w = P.random_weights(cfg, 5)
    folder = U.write_model(str(tmp_path), cfg, w)
    eng = Engine.from_folder(folder, dtype="float32", max_slots=4, max_context=64)
    prompts = [U.random_tokens(n, 5003, 200 + i) for i, n in enumerate((3, 9, 17, 6))]
    sps = [SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True),
           SamplingParams(max_tokens=6, temperature=0.9, seed=4, ignore_eos=True),
           SamplingParams(max_tokens=6, temperature=1.1, top_k=7, seed=5, ignore_eos=True),
           SamplingParams(max_tokens=6, temperature=0.8, top_k=50, top_p=0.7, seed=6, ignore_eos=True)]
    got = [r.tokens for r in eng.generate(prompts, sps)]
    assert got == [r.tokens for r in eng.generate(prompts, sps, max_batch=3)]
    for i, sp in enumerate(sps):
        rng = np.random.default_rng([sp.seed if sp.seed is not None else 0, i])
        toks = list(prompts[i])
        for tok in got[i]:
            u = float(rng.random(dtype=np.float32)) if sp.temperature > 0 else 0.0
            logits = P.forward(cfg, w, toks)[-1].float()
            want = P.sample_token(logits, sp.temperature, sp.top_k, sp.top_p, u)
            if tok != want:
                # a draw that falls within rounding of an interval's edge may go to the neighbour
                wts = P.sample_distribution(logits, sp.temperature, sp.top_k, sp.top_p)
                cdf = torch.cumsum(wts, 0) / wts.sum()
                edge = min(abs(float(cdf[tok]) - u), abs(float(cdf[tok - 1]) - u) if tok else 1.0)
                assert float(wts[tok]) > 0 and edge < 1e-4, (i, tok, want)
            toks.append(tok)


def test_command_line_json(model_a):
    cfg, w, folder = model_a
    prompt = [2] + U.random_tokens(6, 512, 110)
    out = subprocess.run([sys.executable, "-m", "agave_amd", folder, " ".join(map(str, prompt)), "-n", "5",
                          "--dtype", "float32", "--json", "--ignore-eos", "--ctx-size", "64", "--max-batch", "2"],
                         capture_output=True, text=True, cwd=ROOT, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    rec = json.loads(out.stdout.strip().splitlines()[-1])
    assert rec["outputs"][0]["tokens"] == plain_greedy(cfg, w, prompt, 5)
    assert rec["tokens"] == 5 and rec["prefill_tokens"] == 7
    for key in ("tok_per_sec", "prefill_ms", "prefill_tok_per_sec", "gen_ms"):      # src/display.zig:702-744
        assert key in rec
    info = subprocess.run([sys.executable, "-m", "agave_amd", folder, "--model-info", "--json", "--dtype", "float32"],
                          capture_output=True, text=True, cwd=ROOT, timeout=600)
    assert info.returncode == 0, info.stderr[-2000:]
    meta = json.loads(info.stdout.strip().splitlines()[-1])
    assert meta["architecture"] == "Gemma3ForCausalLM" and meta["n_layers"] == 4 and meta["vocab_size"] == 512


def test_profile_option_times_every_class_of_op_without_changing_tokens(model_a):
    """--profile (src/main.zig:381): per-op wall time; the tokens are those of an unprofiled run."""
    cfg, w, folder = model_a
    prompt = [2] + U.random_tokens(9, 512, 111)
    out = subprocess.run([sys.executable, "-m", "agave_amd", folder, " ".join(map(str, prompt)), "-n", "6",
                          "--dtype", "bfloat16", "--json", "--ignore-eos", "--ctx-size", "64", "--profile"],
                         capture_output=True, text=True, cwd=ROOT, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    rec = json.loads(out.stdout.strip().splitlines()[-1])
    ops = {r["op"]: r for r in rec["profile"]}
    for part in ("qkv", "attn_o", "gate_up", "ffn_down", "lm_head"):
        assert any(name.endswith(":" + part) for name in ops), (part, sorted(ops))
    assert any(name.startswith("residual_norm") for name in ops) and any("attn" in name for name in ops)
    # the prompt's step: two norms a layer, and at the model's end the last branch's add and the final
    # norm of the wanted row; the five steps of one token: only the model's end, in one kernel (the
    # layers' products make their normalised rows themselves)
    assert ops["residual_norm"]["calls"] == (2 * 4 + 2) + 5 * 1 and all(r["ms"] >= 0 for r in rec["profile"])
    assert ops["gemm_row_normed:qkv"]["calls"] == 5 * 4 and ops["gemm_row_normed:gate_up"]["calls"] == 5 * 4
    plain = subprocess.run([sys.executable, "-m", "agave_amd", folder, " ".join(map(str, prompt)), "-n", "6",
                            "--dtype", "bfloat16", "--json", "--ignore-eos", "--ctx-size", "64"],
                           capture_output=True, text=True, cwd=ROOT, timeout=600)
    assert json.loads(plain.stdout.strip().splitlines()[-1])["outputs"][0]["tokens"] == rec["outputs"][0]["tokens"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_tool_whole_tail_and_batches(model_b, dtype, tmp_path):
    """bin/trace_run as a user calls it: the same requests whole, with the last 32 tokens one by
    one, and in batches of unequal lengths one after another."""
    cfg, w, folder = model_b
    v = cfg["vocab_size"]
    reqs = [U.random_tokens(n, v, 120 + i) for i, n in enumerate((40, 75, 9, 64, 33))]
    refs = [U.plain_logits(cfg, w, r) for r in reqs]

    def check(got, ref, what):
        if dtype == "float32":
            assert float((got - ref).abs().max()) < 3e-5, what
        else:
            assert float(((got - ref).abs().max(-1).values / ref.abs().max(-1).values).max()) < 0.04, what

    # whole, each alone; then tail32, each alone: one request after another in one process
    whole = [[r] for r in reqs]
    rec, where = U.trace_steps_batched(whole, [[len(r)] for r in reqs])
    out = U.run_trace_tool(folder, dtype, rec, str(tmp_path / "whole"), 128, v)
    for i, ref in enumerate(refs):
        got = torch.from_numpy(np.stack([out[s][row] for s, row in where[(i, 0)]])).double()
        check(got, ref, f"whole {i}")
    rec, where = U.trace_steps_batched(whole, [[max(1, len(r) - 32)] for r in reqs])
    out = U.run_trace_tool(folder, dtype, rec, str(tmp_path / "tail"), 128, v)
    for i, ref in enumerate(refs):
        got = torch.from_numpy(np.stack([out[s][row] for s, row in where[(i, 0)]])).double()
        check(got, ref, f"tail {i}")
    # batches of unequal lengths; the cache holds exactly what the live requests need
    batches = [[reqs[0], reqs[1], reqs[2]], [reqs[3], reqs[4]], [reqs[1], reqs[0]]]
    plens = [[30, 60, 2], [64, 1], [75, 8]]
    rec, where = U.trace_steps_batched(batches, plens)
    need = max(sum(-(-len(r) // 64) * 64 for r in b) for b in batches)
    out = U.run_trace_tool(folder, dtype, rec, str(tmp_path / "batched"), need, v)
    for bi, b in enumerate(batches):
        for ri, r in enumerate(b):
            got = torch.from_numpy(np.stack([out[s][row] for s, row in where[(bi, ri)]])).double()
            check(got, U.plain_logits(cfg, w, r), f"batch {bi} request {ri}")
    # a step that wants nothing writes no file
    assert not os.path.exists(str(tmp_path / "none" / "0.f32"))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_tool_cuts_whole_requests_itself(dtype, tmp_path):
    """bin/trace_run --trace FILE --mode whole|tail32|batched on a model it makes itself from a
    configuration and a seed (random:CONFIG.json:SEED): every mode gives each request's logits at
    every position, equal to the plain implementation's on the weights the tool wrote."""
    from agave_amd.weights import Checkpoint
    cfg = P.tiny_config("A")
    cfg_path = str(tmp_path / "cfg.json")
    with open(cfg_path, "w") as f:
        json.dump(cfg, f)
    v = cfg["vocab_size"]
    lens = (50, 70, 5, 41)
    reqs = [{"id": f"r{i}", "tokens": U.random_tokens(n, v, 500 + i), "prompt": p, "batch": i // 3}
            for i, (n, p) in enumerate(zip(lens, (20, 64, 1, 41)))]
    trace = str(tmp_path / "trace.jsonl")
    with open(trace, "w") as f:
        for r in reqs:
            f.write(json.dumps(r) + "\n")
    refs = None
    for mode in ("whole", "tail32", "batched"):
        out = str(tmp_path / mode)
        proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", f"random:{cfg_path}:5",
                               "--dtype", dtype, "--out", out, "--trace", trace, "--mode", mode],
                              capture_output=True, text=True, timeout=600)
        assert proc.returncode == 0, proc.stderr[-3000:]
        if refs is None:
            ck = Checkpoint(os.path.join(out, "model"))
            w = {n: ck.read(n).double() for n in ck.names()}
            refs = [U.plain_logits(cfg, w, r["tokens"]) for r in reqs]
        index = json.load(open(os.path.join(out, "index.json")))
        assert index["mode"] == mode and sorted(index["requests"]) == [r["id"] for r in reqs]
        steps = [int(l.split()[1]) for l in proc.stdout.splitlines() if l.startswith("done ")]
        assert steps == list(range(len(steps)))
        # whole: a step a request; tail32: one and its tail each; batched: two batches, the longest request sets the steps
        assert len(steps) == {"whole": 4, "tail32": sum(1 + min(32, n - 1) for n in lens),
                              "batched": (1 + max(50 - 20, 70 - 64, 5 - 1)) + 1}[mode]
        for r, ref in zip(reqs, refs):
            meta = index["requests"][r["id"]]
            got = torch.from_numpy(np.fromfile(os.path.join(out, meta["file"]), dtype="<f4").reshape(meta["positions"], meta["vocab"])).double()
            assert got.shape == ref.shape
            if dtype == "float32":
                assert float((got - ref).abs().max()) < 3e-5, (mode, r["id"])
            else:
                assert float(((got - ref).abs().max(-1).values / ref.abs().max(-1).values).max()) < 0.04, (mode, r["id"])


def test_steps_launched_ahead_give_the_tokens_of_steps_run_one_by_one(model_b):
    """launch_step with tokens carried on the device (also for a shrinking subset of the rows, in
    another order) against step_sample fed from the host."""
    from agave_amd.engine import Engine
    from agave_amd.engine.generate import RowSampling
    cfg, w, folder = model_b
    a = Engine.from_folder(folder, dtype="float32", max_slots=4, max_context=96)
    b = Engine.from_folder(folder, dtype="float32", max_slots=4, max_context=96)
    prompts = [U.random_tokens(n, cfg["vocab_size"], 300 + i) for i, n in enumerate((9, 1, 30, 14))]
    rows = lambda k: [RowSampling(0.0, 0, 1.0, 1.0, 0.0, []) for _ in range(k)]
    sa = [a.alloc_slot() for _ in prompts]
    sb = [b.alloc_slot() for _ in prompts]
    keep = [[0, 1, 2, 3], [0, 1, 2, 3], [3, 0, 2], [3, 0, 2], [2, 3], [2], [2]]     # rows of the first step, per step
    # one by one, from the host
    toks = a.step_sample(sa, prompts, rows(4))
    ref = [list(toks)]
    cur = list(range(4))
    for k in keep:
        toks = a.step_sample([sa[i] for i in k], [[toks[cur.index(i)]] for i in k], rows(len(k)))
        cur = k
        ref.append(list(toks))
    # launched ahead, tokens carried on the device
    got = []
    running = b.launch_step(sb, prompts, rows(4))
    cur = list(range(4))
    for k in keep:
        following = b.launch_step([sb[i] for i in k], None, rows(len(k)), [cur.index(i) for i in k])
        got.append(b.finish_step(running))
        running, cur = following, k
    got.append(b.finish_step(running))
    assert got == ref


def test_repeat_penalty_through_the_engine(model_a):
    """Requests of one batch with different penalties (one without): every token is the plain
    argmax of the plain logits after the plain penalty over that request's own generated ids.  The
    prompts end in a token that greedy decoding repeats, so the penalty changes what comes out."""
    from agave_amd import Engine, SamplingParams
    cfg, w, folder = model_a
    eng = Engine.from_folder(folder, dtype="float32", max_slots=3, max_context=64)
    prompts = [U.random_tokens(n, 512, 400 + i) for i, n in enumerate((7, 12, 3))]
    penalties = [1.3, 1.0, 2.5]
    sps = [SamplingParams(max_tokens=14, repeat_penalty=p, ignore_eos=True) for p in penalties]
    got = [r.tokens for r in eng.generate(prompts, sps)]
    free = [r.tokens for r in eng.generate(prompts, SamplingParams(max_tokens=14, ignore_eos=True))]
    for i, (prompt, pen) in enumerate(zip(prompts, penalties)):
        toks, out = list(prompt), []
        for _ in range(14):
            logits = P.apply_repeat_penalty(P.forward(cfg, w, toks)[-1], out, pen)
            out.append(P.argmax_first(logits))
            toks.append(out[-1])
        assert got[i] == out, f"request {i} with penalty {pen}"
    assert got[1] == free[1]
    assert got[0] != free[0] or got[2] != free[2], "the penalty changed nothing: the test proves nothing"
    # the same requests alone and in another order: the ids and rows of a penalty belong to its request
    again = [r.tokens for r in eng.generate(prompts[::-1], sps[::-1], max_batch=2)]
    assert again == got[::-1]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_more_kinds_of_decode_steps_than_graphs_are_kept(model_b, dtype):
    """Twenty requests with twenty different lengths: the batch shrinks by one request every three
    steps, so twenty kinds of decode step pass by while four graphs are kept.  Old graphs make room,
    every kind of step is still recorded, and the tokens are those of an engine without graphs."""
    from agave_amd import Engine, SamplingParams
    cfg, w, folder = model_b
    v = cfg["vocab_size"]
    a = Engine.from_folder(folder, dtype=dtype, max_slots=20, max_context=128)
    b = Engine.from_folder(folder, dtype=dtype, max_slots=20, max_context=128)
    a.graphs.max_graphs = 4
    b.use_graphs = False
    prompts = [U.random_tokens(1 + (5 * i) % 23, v, 500 + i) for i in range(20)]
    sps = [SamplingParams(max_tokens=4 + 3 * i, ignore_eos=True) for i in range(20)]
    ra = a.generate(prompts, sps)
    rb = b.generate(prompts, sps)
    assert [r.tokens for r in ra] == [r.tokens for r in rb]
    assert all(len(r.tokens) == 4 + 3 * i for i, r in enumerate(ra))
    kept = list(a.graphs._graphs)
    assert len(kept) <= 4 and a.graphs.evicted >= 14
    assert sorted(k[0] for k in kept) == [1, 2, 3, 4], kept          # the batch sizes that ran last
    assert not b.graphs._graphs


def test_log_probabilities_of_the_generated_tokens(model_b):
    """Requests that ask for them get, with every emitted token, the natural logarithm of the model's
    probability of that token (from the logits as the sampler saw them), whatever way it was drawn
    and whether steps run ahead or not; a stop token is not emitted and neither is its number."""
    import math
    from agave_amd import Engine, SamplingParams
    cfg, w, folder = model_b
    eng = Engine.from_folder(folder, dtype="float32", max_slots=3, max_context=96)
    prompts = [U.random_tokens(n, cfg["vocab_size"], 600 + i) for i, n in enumerate((4, 21, 9))]
    sps = [SamplingParams(max_tokens=7, logprobs=True, ignore_eos=True),
           SamplingParams(max_tokens=5, temperature=0.9, seed=3, ignore_eos=True),                      # does not ask
           SamplingParams(max_tokens=6, temperature=1.3, top_k=20, seed=4, logprobs=True, ignore_eos=True)]
    res = eng.generate(prompts, sps)
    assert res[1].logprobs == [] and len(res[0].logprobs) == 7 and len(res[2].logprobs) == 6
    for i in (0, 2):
        toks = list(prompts[i])
        for tok, lp in zip(res[i].tokens, res[i].logprobs):
            row = P.forward(cfg, w, toks)[-1].double()
            want = float(row[tok] - torch.logsumexp(row, 0))
            assert math.isclose(lp, want, rel_tol=0, abs_tol=2e-4), (i, len(toks), lp, want)
            toks.append(tok)
    # with a repeat penalty (steps do not run ahead then) and a stop token
    stop = res[0].tokens[3]
    one = eng.generate([prompts[0]], SamplingParams(max_tokens=7, logprobs=True, repeat_penalty=1.0, stop_ids=(stop,)))[0]
    assert one.finish_reason == "stop" and one.tokens == res[0].tokens[:3] and len(one.logprobs) == 3
    assert all(math.isclose(a, b, abs_tol=1e-5) for a, b in zip(one.logprobs, res[0].logprobs))
    pen = eng.generate([prompts[0]], SamplingParams(max_tokens=4, logprobs=True, repeat_penalty=1.4, ignore_eos=True))[0]
    toks, out = list(prompts[0]), []
    for tok, lp in zip(pen.tokens, pen.logprobs):
        row = P.apply_repeat_penalty(P.forward(cfg, w, toks)[-1], out, 1.4).double()
        assert tok == P.argmax_first(row) and math.isclose(lp, float(row[tok] - torch.logsumexp(row, 0)), abs_tol=2e-4)
        toks.append(tok)
        out.append(tok)
