"""The engine against the plain implementation on the GPU: each request alone and whole, with
the last 32 tokens one by one, and in batches of unequal lengths whose shorter requests end
earlier, one batch after another so that slots and pages are used again; in 32-bit and in
bfloat16."""
import pytest
import torch

import engine_utils as U
import plain_gemma3 as P

pytestmark = pytest.mark.gpu

# 32-bit: rounding only.  The logits are O(1); a fault in any formula shows as >= 1e-3.
F32_ATOL, F32_RTOL = 2e-5, 1e-5


def bf16_close(got: torch.Tensor, ref: torch.Tensor, what: str):
    """bfloat16 keeps 8 bits: activations are rounded at ~2^-9 relative at each of a few dozen
    places, so a logit row may differ by a few percent of its largest entry."""
    scale = ref.abs().max(dim=-1, keepdim=True).values
    err = ((got.double() - ref) .abs() / scale).max(dim=-1).values
    worst = int(err.argmax())
    assert float(err.max()) < 0.04, f"{what}: relative error {float(err.max()):.4f} at position {worst}"


def f32_close(got: torch.Tensor, ref: torch.Tensor, what: str, longer_sums: float = 1.0):
    """``longer_sums``: how many times longer the model's dot products are than the tiny
    configurations' (a few hundred terms); the rounding error of a 32-bit sum grows with the
    root of its length."""
    diff = (got.double() - ref).abs()
    tol = (F32_ATOL + F32_RTOL * ref.abs()) * longer_sums ** 0.5
    bad = (diff > tol).any(dim=-1)
    if bad.any():
        first = int(torch.nonzero(bad)[0])
        raise AssertionError(f"{what}: first wrong position {first} of {got.shape[0]}, "
                             f"max error there {float(diff[first].max()):.3e}, overall {float(diff.max()):.3e}")


def close(dtype):
    return f32_close if dtype == "float32" else bf16_close


@pytest.fixture(scope="module", params=["A", "B", "C"])
def tiny(request, tmp_path_factory):
    which = request.param
    cfg = P.tiny_config(which)
    weights = P.random_weights(cfg, {"A": 0, "B": 1, "C": 2}[which])
    folder = U.write_model(str(tmp_path_factory.mktemp(f"tiny{which}")), cfg, weights)
    return which, cfg, weights, folder


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def engine_of(request, tiny):
    from agave_amd.engine import Engine
    which, cfg, weights, folder = tiny
    eng = Engine.from_folder(folder, dtype=request.param, max_slots=6, max_context=192)
    return eng, request.param, cfg, weights


def test_whole_prompt(engine_of):
    eng, dtype, cfg, weights = engine_of
    for n, seed in ((1, 10), (5, 11), (40, 12), (150, 13)):
        toks = U.random_tokens(n, cfg["vocab_size"], seed)
        close(dtype)(U.run_whole(eng, toks), U.plain_logits(cfg, weights, toks), f"whole n={n}")


def test_tail_one_by_one(engine_of):
    eng, dtype, cfg, weights = engine_of
    for n, seed in ((33, 20), (100, 21), (160, 22)):
        toks = U.random_tokens(n, cfg["vocab_size"], seed)
        ref = U.plain_logits(cfg, weights, toks)
        close(dtype)(U.run_tail(eng, toks, 32), ref, f"tail n={n}")


def test_first_tokens_one_by_one(engine_of):
    eng, dtype, cfg, weights = engine_of
    toks = U.random_tokens(20, cfg["vocab_size"], 30)
    close(dtype)(U.run_tail(eng, toks, 19), U.plain_logits(cfg, weights, toks), "from the first token")


def test_batches_of_unequal_lengths_reuse_slots(engine_of):
    eng, dtype, cfg, weights = engine_of
    v = cfg["vocab_size"]
    batches = [
        ([U.random_tokens(n, v, 40 + i) for i, n in enumerate((13, 48, 27))], (5, 40, 19)),
        ([U.random_tokens(n, v, 50 + i) for i, n in enumerate((9, 70, 31, 69, 100))], (1, 57, 13, 30, 7)),
        ([U.random_tokens(n, v, 60 + i) for i, n in enumerate((66, 3))], (64, 3)),
    ]
    for bi, (reqs, plens) in enumerate(batches):
        outs = U.run_batched(eng, reqs, plens)
        for i, (r, o) in enumerate(zip(reqs, outs)):
            close(dtype)(o, U.plain_logits(cfg, weights, r), f"batch {bi} request {i}")
    assert eng.cache.slots.n_free == eng.cache.max_slots
    for g in eng.cache.groups:
        assert g.pool.n_free == g.pool.n_pages


def test_cutting_gives_the_same_numbers(engine_of):
    """With the plain kernels a position's arithmetic does not depend on the cutting at all;
    with the matrix-core kernels it may differ by rounding."""
    eng, dtype, cfg, weights = engine_of
    toks = U.random_tokens(90, cfg["vocab_size"], 70)
    whole, tail = U.run_whole(eng, toks), U.run_tail(eng, toks, 32)
    other = U.random_tokens(50, cfg["vocab_size"], 71)
    batched = U.run_batched(eng, [other, toks], (20, 58))[1]
    tol = 1e-5 if dtype == "float32" else 0.03
    scale = float(whole.abs().max())
    assert float((whole - tail).abs().max()) <= tol * scale
    assert float((whole - batched).abs().max()) <= tol * scale


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_equal_eager_steps(tiny, dtype):
    """Decode steps are recorded into a HIP graph on their second occurrence.  Every replay, with
    eager steps of other batches and synchronisations in between, must give what an engine
    without graphs gives."""
    from agave_amd.engine import Engine
    which, cfg, weights, folder = tiny
    a = Engine.from_folder(folder, dtype=dtype, max_slots=4, max_context=256)
    b = Engine.from_folder(folder, dtype=dtype, max_slots=4, max_context=256)
    b.use_graphs = False
    v = cfg["vocab_size"]
    prompts = [U.random_tokens(n, v, 200 + i) for i, n in enumerate((70, 3, 129))]
    sa = [a.alloc_slot() for _ in prompts]
    sb = [b.alloc_slot() for _ in prompts]
    a.step(sa, prompts, "last")
    b.step(sb, prompts, "last")
    other = a.alloc_slot()
    for i in range(70):                       # crosses page boundaries and, for window 70, its edge
        toks = [[(7 * i + 3 * j) % v] for j in range(3)]
        la = a.step(sa, toks, "last").clone()
        lb = b.step(sb, toks, "last").clone()
        assert torch.equal(la, lb), f"step {i}"
        if i % 9 == 0:                        # eager work of another sequence between replays
            a.step([other], [U.random_tokens(5, v, i)], "last")
            torch.cuda.synchronize()
    assert len(a.graphs._graphs) >= 1


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_short_prompts_of_one_sequence_are_replayed_as_graphs(tiny, dtype):
    """A short prompt of one sequence that wants its last row is padded until it ends at a multiple
    of 16 positions and, from its kind's second occurrence on, recorded and replayed.  Prompts of
    different lengths that end in the same stretch share a graph: each must give what the plain
    implementation gives for its own length, on the eager run, on the recording and on every
    replay, and so must the tokens decoded after it (they come to stand where the padding left
    keys and values), also when the prompt is a continuation that starts in the middle of a page."""
    from agave_amd.engine import Engine
    from agave_amd.engine.graphs import PROMPT_GRAPH_PAD, PROMPT_GRAPH_TOKENS
    assert (PROMPT_GRAPH_PAD, PROMPT_GRAPH_TOKENS) == (16, 128)      # the lengths below are chosen for these
    which, cfg, weights, folder = tiny
    eng = Engine.from_folder(folder, dtype=dtype, max_slots=3, max_context=256)
    v = cfg["vocab_size"]
    seed = 300
    # (a long one first: it sizes the workspace, and it is too long to be recorded)
    for lengths in ((150,), (100, 112, 97, 105), (5, 16, 2, 9), (60, 64, 49), (128, 113, 120)):
        for n in lengths:
            seed += 1
            toks = U.random_tokens(n + 4, v, seed)
            ref = U.plain_logits(cfg, weights, toks)
            slot = eng.alloc_slot()
            got = [eng.step([slot], [toks[:n]], "last").float().cpu().clone()]
            for t in toks[n:]:
                got.append(eng.step([slot], [[t]], "last").float().cpu().clone())
            eng.free_slot(slot)
            close(dtype)(torch.cat(got, 0), ref[n - 1:], f"prompt of {n} and four tokens after it")
    kinds = [k for k in eng.graphs._graphs if k[0] == "prompt"]
    assert sorted(k[1] for k in kinds) == [16, 64, 112, 128], kinds

    # continuations: 40 tokens, then some more that end between 81 and 96 (a step that starts at 40 and is
    # padded to 56 rows), three times so that it is run eagerly, recorded and replayed
    for rep, more in enumerate((50, 56, 41)):
        toks = U.random_tokens(40 + more + 3, v, 400 + rep)
        ref = U.plain_logits(cfg, weights, toks)
        slot = eng.alloc_slot()
        got = [eng.step([slot], [toks[:40]], "last").float().cpu().clone(),
               eng.step([slot], [toks[40:40 + more]], "last").float().cpu().clone()]
        for t in toks[40 + more:]:
            got.append(eng.step([slot], [[t]], "last").float().cpu().clone())
        eng.free_slot(slot)
        want = torch.cat([ref[39:40], ref[40 + more - 1:]], 0)
        close(dtype)(torch.cat(got, 0), want, f"40 tokens, then {more} more")
    assert any(k[0] == "prompt" and k[1:3] == (56, 40) for k in eng.graphs._graphs)
    for g in eng.cache.groups:
        assert g.pool.n_free == g.pool.n_pages


def test_long_decoding(engine_of):
    """A short prompt, then many tokens one by one: over page edges, past the window's reach (the
    window groups give pages back while the sequence grows) and through many graph replays."""
    eng, dtype, cfg, weights = engine_of
    toks = U.random_tokens(190, cfg["vocab_size"], 80)
    ref = U.plain_logits(cfg, weights, toks)
    close(dtype)(U.run_tail(eng, toks, 183), ref, "long decoding")
    for g in eng.cache.groups:
        assert g.pool.n_free == g.pool.n_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_context_of_thousands_of_tokens(tmp_path, dtype):
    """Dozens of pages a sequence and a window that reaches over two dozen of them: the prompt
    whole, then in three pieces beside a short request, then further tokens one by one; the
    long dot products of attention over thousands of keys are where a lost page would show."""
    from agave_amd.engine import Engine
    cfg = dict(P.tiny_config("C"))
    cfg["sliding_window"] = 1500
    weights = P.random_weights(cfg, 5)
    folder = U.write_model(str(tmp_path / "m"), cfg, weights)
    eng = Engine.from_folder(folder, dtype=dtype, max_slots=2, max_context=4224)
    long_req = U.random_tokens(4200, cfg["vocab_size"], 7)
    short_req = U.random_tokens(70, cfg["vocab_size"], 8)
    ref = U.plain_logits(cfg, weights, long_req)
    check = close(dtype)
    kw = dict(longer_sums=8.0) if dtype == "float32" else {}
    check(U.run_whole(eng, long_req[:4100]), ref[:4100], "whole", **kw)
    slots = [eng.alloc_slot(), eng.alloc_slot()]
    got = []
    for lo, hi, slo, shi in ((0, 2048, 0, 30), (2048, 4095, 30, 31), (4095, 4160, 31, 70)):
        lg = eng.step(slots, [long_req[lo:hi], short_req[slo:shi]], "all").float().cpu()
        got.append(lg[:hi - lo].clone())
    eng.free_slot(slots[1])
    for t in long_req[4160:]:
        got.append(eng.step(slots[:1], [[t]], "all").float().cpu().clone())
    eng.free_slot(slots[0])
    check(torch.cat(got, 0), ref, "pieces, then one by one", **kw)
    for g in eng.cache.groups:
        assert g.pool.n_free == g.pool.n_pages


def test_prompt_in_pieces(engine_of):
    """Steps of several tokens that start in the middle of a sequence (a prompt that enters in
    pieces): pieces that end on a page's edge, one short of it and one past it, for two
    sequences of unequal lengths at once."""
    eng, dtype, cfg, weights = engine_of
    v = cfg["vocab_size"]
    reqs = [U.random_tokens(170, v, 90), U.random_tokens(131, v, 91)]
    cuts = [(0, 63, 64, 129, 170), (0, 1, 65, 128, 131)]
    slots = [eng.alloc_slot() for _ in reqs]
    outs = [[], []]
    for piece in range(4):
        chunks = [r[c[piece]:c[piece + 1]] for r, c in zip(reqs, cuts)]
        logits = eng.step(slots, chunks, "all").float().cpu()
        o = 0
        for i, ch in enumerate(chunks):
            outs[i].append(logits[o:o + len(ch)].clone())
            o += len(ch)
    for s in slots:
        eng.free_slot(s)
    for i, r in enumerate(reqs):
        close(dtype)(torch.cat(outs[i], 0), U.plain_logits(cfg, weights, r), f"request {i} in pieces")


def _save_folder(folder, cfg, stored):
    from safetensors.torch import save_file
    import json, os
    os.makedirs(folder)
    save_file({k: v.contiguous() for k, v in stored.items()}, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    return folder


def test_tensors_stored_in_32_bit_stay_so_in_a_bfloat16_engine(tmp_path):
    """A checkpoint that stores some matrices, a norm and the output matrix in 32-bit, with values
    that bfloat16 cannot hold: the bfloat16 engine keeps them in 32-bit and gives the plain logits.
    The output matrix is made so that rounding it would show: every row is the same vector of +-1
    plus a small part of its own, which bfloat16 drops (its steps near 1 are 2^-8 and 2^-7).  What
    tells the vocabulary's entries apart then lies in the dropped part alone, so the logits minus
    their mean over the vocabulary are right only if the 32-bit values took part.  An engine on the
    same tensors rounded to bfloat16 first matches its own plain logits and not the other's."""
    from agave_amd.engine import Engine
    cfg = P.tiny_config("C")                       # untied output matrix
    weights = P.random_weights(cfg, 7, bf16_exact=False)
    g = torch.Generator().manual_seed(3)
    sign = (torch.randint(0, 2, (cfg["hidden_size"],), generator=g) * 2 - 1).double()
    weights["lm_head.weight"] = sign[None, :] + 0.002 * torch.randn(cfg["vocab_size"], cfg["hidden_size"],
                                                                     generator=g, dtype=torch.float64)
    kept32 = [k for k in weights if k.endswith(("lm_head.weight", "q_proj.weight", "down_proj.weight",
                                                "input_layernorm.weight"))]
    assert any((weights[k].bfloat16().double() != weights[k].float().double()).any() for k in kept32)
    stored = {k: (v.float() if k in kept32 else v.bfloat16()) for k, v in weights.items()}
    rounded = {k: v.bfloat16() for k, v in weights.items()}
    toks = U.random_tokens(70, cfg["vocab_size"], 5)
    ref = U.plain_logits(cfg, {k: v.double() for k, v in stored.items()}, toks)
    ref_rounded = U.plain_logits(cfg, {k: v.double() for k, v in rounded.items()}, toks)

    def centred(x):
        x = x.double()
        return x - x.mean(dim=-1, keepdim=True)

    def apart(a, b):
        """Largest difference of two sets of centred logits, in units of the first one's spread."""
        return float(((centred(a) - centred(b)).abs().max(dim=-1).values / centred(a).abs().max(dim=-1).values).max())

    def common_close(got, want, what):
        """The part that all entries of a row share is a sum of +-x_j over the final row x, which
        cancels to anything between 0 and a dozen: its error is measured against the length of x
        (about sqrt(hidden)), not against the sum itself."""
        err = (got.double().mean(-1) - want.mean(-1)).abs().max()
        assert float(err) < 0.04 * cfg["hidden_size"] ** 0.5, f"{what}: common part off by {float(err):.3f}"

    assert apart(ref, ref_rounded) > 0.5            # the construction works: rounding changes what is compared
    eng = Engine.from_folder(_save_folder(str(tmp_path / "mixed"), cfg, stored), dtype="bfloat16", max_slots=2,
                             max_context=128)
    attn0 = eng.model.blocks[0].mixer
    assert attn0.qkv.packed is None and attn0.qkv.weight.dtype == torch.float32
    assert eng.model.head.packed is None and eng.model.head.weight.dtype == torch.float32
    assert eng.model.blocks[0].ffn.gate_up.packed is not None          # stored in bfloat16: on the matrix cores
    whole, tail = U.run_whole(eng, toks), U.run_tail(eng, toks, 20)
    common_close(whole, ref, "mixed storage, whole")
    common_close(tail, ref, "mixed storage, tail")
    assert apart(ref, whole) < 0.1 and apart(ref, tail) < 0.1
    del eng
    eng = Engine.from_folder(_save_folder(str(tmp_path / "rounded"), cfg, rounded), dtype="bfloat16", max_slots=2,
                             max_context=128)
    assert eng.model.head.packed is not None
    got = U.run_whole(eng, toks)
    common_close(got, ref_rounded, "rounded storage")
    assert apart(ref_rounded, got) < 0.1 and apart(ref, got) > 0.5
    del eng
    # told to cast, the engine on the 32-bit folder behaves as the one on the rounded folder
    eng = Engine.from_folder(str(tmp_path / "mixed"), dtype="bfloat16", max_slots=2, max_context=128,
                             keep_stored_precision=False)
    assert eng.model.head.packed is not None and eng.model.blocks[0].mixer.qkv.packed is not None
    got = U.run_whole(eng, toks)
    assert apart(ref_rounded, got) < 0.1 and apart(ref, got) > 0.5


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_a_half_precision_folder_is_cast_to_the_engine_s_type(tmp_path, dtype):
    """Every tensor stored as F16: a bfloat16 engine casts the matrices to bfloat16 and runs them on
    the matrix cores, a 32-bit engine widens them exactly."""
    from agave_amd.engine import Engine
    cfg = P.tiny_config("C")
    weights = P.random_weights(cfg, 8)
    stored = {k: v.half() for k, v in weights.items()}
    eng = Engine.from_folder(_save_folder(str(tmp_path / "half"), cfg, stored), dtype=dtype, max_slots=2,
                             max_context=128)
    qkv = eng.model.blocks[0].mixer.qkv
    if dtype == "bfloat16":
        assert qkv.packed is not None and eng.model.head.packed is not None and not eng.env.kept_32bit
    else:
        assert qkv.weight.dtype == torch.float32
    toks = U.random_tokens(70, cfg["vocab_size"], 6)
    as_held = {k: (v.bfloat16() if dtype == "bfloat16" and v.dim() == 2 else v).double() for k, v in stored.items()}
    ref = U.plain_logits(cfg, as_held, toks)
    close(dtype)(U.run_whole(eng, toks), ref, "half-precision storage, whole")
    close(dtype)(U.run_tail(eng, toks, 20), ref, "half-precision storage, tail")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("prefix", ["language_model.model.", "model.language_model."])
def test_a_folder_that_holds_more_than_the_decoder(tmp_path, dtype, prefix):
    """A folder in the layout of the published checkpoints: the text keys inside ``text_config``,
    the decoder's tensors under a prefix, a vision tower and a projector beside them
    (src/format/safetensors.zig:333-349, 517-521; src/arch.zig:22-23).  The logits are the plain
    implementation's of the decoder alone."""
    from agave_amd.engine import Engine
    inner = P.tiny_config("A")
    weights = P.random_weights(inner, 4)
    raw = {"architectures": ["Gemma3ForConditionalGeneration"], "model_type": "gemma3",
           "text_config": {k: v for k, v in inner.items() if k != "architectures"},
           "vision_config": {"hidden_size": 8}}
    stored = {prefix + k[len("model."):]: v.bfloat16() for k, v in weights.items()}
    stored["vision_tower.vision_model.embeddings.patch_embedding.weight"] = torch.randn(4, 3, 2, 2).bfloat16()
    stored["multi_modal_projector.mm_input_projection_weight"] = torch.randn(8, 8).bfloat16()
    eng = Engine.from_folder(_save_folder(str(tmp_path / "wrapped"), raw, stored), dtype=dtype, max_slots=2,
                             max_context=128)
    toks = U.random_tokens(60, inner["vocab_size"], 12)
    ref = U.plain_logits(inner, weights, toks)
    close(dtype)(U.run_whole(eng, toks), ref, "wrapped folder, whole")
    close(dtype)(U.run_tail(eng, toks, 20), ref, "wrapped folder, tail")


def _fast_head_config(head_dim, n_heads, n_kv, window, pattern):
    """A narrow model whose heads take the kernels for head sizes 64, 128 and 256."""
    cfg = dict(P.tiny_config("A"), vocab_size=640, hidden_size=128, num_hidden_layers=3, num_attention_heads=n_heads,
               num_key_value_heads=n_kv, head_dim=head_dim, query_pre_attn_scalar=head_dim, intermediate_size=320,
               sliding_window=window, sliding_window_pattern=pattern, rope_theta=1e6, rope_local_base_freq=1e4,
               rope_scaling={"rope_type": "linear", "factor": 4.0}, rms_norm_eps=1e-6, max_position_embeddings=4096)
    cfg.pop("layer_types", None)
    return cfg


@pytest.mark.parametrize("which,dtype", [("A", "float32"), ("C", "float32"), ("B", "bfloat16"),
                                         ("heads of 64 in groups of 4", "bfloat16"), ("heads of 256", "bfloat16"),
                                         ("heads of 128", "float32")])
def test_random_schedules_of_ragged_steps(tmp_path, which, dtype):
    """Steps whose make-up is drawn at random: some sequences bring many tokens and others one in
    the same step, sequences start and end at any time, slots and pages are used again, and pieces
    end anywhere relative to page edges and the window.  Every logit row is checked.  The tiny
    configurations run forty steps of up to four sequences of up to 190 tokens; the ones with
    heads of 64, 128 and 256 (the kernels that the published sizes take: prompts by items, decode
    steps with the keys shared among workgroups, the output product that merges their shares)
    sixty steps of up to six sequences of up to 600 tokens, half of them decode steps."""
    import random
    from agave_amd.engine import Engine
    fast = {"heads of 64 in groups of 4": (64, 8, 2, 64, 2), "heads of 256": (256, 2, 1, 130, 3),
            "heads of 128": (128, 4, 2, 100, 2)}.get(which)
    cfg = _fast_head_config(*fast) if fast else P.tiny_config(which)
    weights = {k: v.double() for k, v in P.random_weights(cfg, 3).items()}
    folder = U.write_model(str(tmp_path / "m"), cfg, weights)
    most, context, lengths, pieces, steps = (6, 640, [1, 2, 63, 64, 65, 100, 130, 190, 257, 400, 600],
                                             [1, 3, 31, 64, 70, 129, 300], 60) if fast else \
                                            (4, 200, [1, 2, 63, 64, 65, 100, 130, 190], [1, 3, 31, 64, 70], 40)
    eng = Engine.from_folder(folder, dtype=dtype, max_slots=most, max_context=context)
    rnd = random.Random(17)
    live = {}                       # slot -> [tokens, reference logits, fed so far]
    started = 0
    for it in range(steps):
        while len(live) < most and (started < 3 or not live or rnd.random() < 0.5):
            n = rnd.choice(lengths)
            toks = U.random_tokens(n, cfg["vocab_size"], 1000 + started)
            live[eng.alloc_slot()] = [toks, U.plain_logits(cfg, weights, toks), 0]
            started += 1
        chosen = [s for s in live if rnd.random() < 0.8] or list(live)[:1]
        decode_only = bool(fast) and rnd.random() < 0.5
        chunks = []
        for s in chosen:
            toks, _, fed = live[s]
            room = len(toks) - fed
            k = 1 if (decode_only or rnd.random() < 0.4) else rnd.choice(pieces)
            chunks.append(toks[fed:fed + min(k, room)])
        logits = eng.step(chosen, chunks, "all").float().cpu()
        o = 0
        for s, ch in zip(chosen, chunks):
            toks, ref, fed = live[s]
            close(dtype)(logits[o:o + len(ch)], ref[fed:fed + len(ch)], f"step {it}, slot {s}, positions {fed}..{fed + len(ch) - 1}")
            o += len(ch)
            live[s][2] = fed + len(ch)
            if live[s][2] == len(toks):
                eng.free_slot(s)
                del live[s]
    for s in list(live):
        eng.free_slot(s)
    assert eng.cache.slots.n_free == eng.cache.max_slots
    for g in eng.cache.groups:
        assert g.pool.n_free == g.pool.n_pages


BIG_LAYERS = {
    # the 4B model's layers: width 2560, 8 query and 4 kv heads of 256, 10240 inner columns, window 1024
    "4b": (dict(hidden_size=2560, num_attention_heads=8, num_key_value_heads=4, head_dim=256, query_pre_attn_scalar=256,
                intermediate_size=10240, sliding_window=1024), 1060, 1015),
    # the 12B model's: width 3840, 16 query and 8 kv heads of 256, 15360 inner columns (other cuts of the
    # row blocks among workgroups than the 4B sizes'); a shorter window, as for the 27B sizes
    "12b": (dict(hidden_size=3840, num_attention_heads=16, num_key_value_heads=8, head_dim=256,
                 query_pre_attn_scalar=256, intermediate_size=15360, sliding_window=256), 300, 250),
    # the 27B model's: width 5376, 32 query and 16 kv heads of 128, a scale that is not the head size;
    # a shorter window so that the plain implementation stays quick
    "27b": (dict(hidden_size=5376, num_attention_heads=32, num_key_value_heads=16, head_dim=128,
                 query_pre_attn_scalar=168, intermediate_size=21504, sliding_window=256), 300, 250),
}


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("size", sorted(BIG_LAYERS))
def test_layers_of_the_published_sizes(tmp_path, dtype, size):
    """Two layers with a published model's own sizes (the second one global with its scaled rope) and
    a small vocabulary: a prompt that ends just short of the window's reach, then steps across it;
    then three requests of unequal lengths as one batch whose shorter ones end earlier."""
    from agave_amd.engine import Engine
    sizes, n_all, n_prompt = BIG_LAYERS[size]
    cfg = dict(P.tiny_config("A"), vocab_size=1536, num_hidden_layers=2, sliding_window_pattern=2, rope_theta=1e6,
               rope_local_base_freq=1e4, rope_scaling={"rope_type": "linear", "factor": 8.0}, rms_norm_eps=1e-6,
               max_position_embeddings=4096, **sizes)
    cfg.pop("layer_types", None)
    weights = P.random_weights(cfg, 11)
    folder = U.write_model(str(tmp_path / "m"), cfg, weights)
    eng = Engine.from_folder(folder, dtype=dtype, max_slots=3, max_context=1152)
    toks = U.random_tokens(n_all, cfg["vocab_size"], 12)
    ref = U.plain_logits(cfg, weights, toks)
    first = [0, 1, n_prompt // 2, n_prompt - 2, n_prompt - 1]
    slot = eng.alloc_slot()
    got = [eng.step([slot], [toks[:n_prompt]], [first]).float().cpu().clone()]
    for t in toks[n_prompt:]:
        got.append(eng.step([slot], [[t]], "last").float().cpu().clone())
    eng.free_slot(slot)
    rows = first + list(range(n_prompt, len(toks)))
    kw = dict(longer_sums=sizes["intermediate_size"] / 320) if dtype == "float32" else {}
    close(dtype)(torch.cat(got, 0), ref[rows], f"{size} layers", **kw)
    others = [U.random_tokens(n, cfg["vocab_size"], 13 + i) for i, n in enumerate((150, 67))]
    outs = U.run_batched(eng, [toks] + others, (n_prompt - 9, 120, 3))
    close(dtype)(outs[0], ref, f"{size} layers, first of a batch", **kw)
    for i, (r, o) in enumerate(zip(others, outs[1:])):
        close(dtype)(o, U.plain_logits(cfg, weights, r), f"{size} layers, request {i + 1} of a batch", **kw)


@pytest.mark.parametrize("n_seqs", [12, 70])
def test_wide_batches_at_a_published_size(tmp_path, n_seqs):
    """Decode steps of 12 and of 70 sequences with the 4B model's layer sizes: the products of 9 to
    16 tokens are cut into workgroups like the larger batches', those of 65 and more run in tiles,
    and the attention's splits follow the number of sequences.  Requests of unequal lengths, so the
    batch shrinks as it goes."""
    from agave_amd.engine import Engine
    sizes, _, _ = BIG_LAYERS["4b"]
    cfg = dict(P.tiny_config("A"), vocab_size=1536, num_hidden_layers=2, sliding_window_pattern=2, rope_theta=1e6,
               rope_local_base_freq=1e4, rms_norm_eps=1e-6, max_position_embeddings=4096, **dict(sizes, sliding_window=24))
    cfg.pop("layer_types", None)
    weights = P.random_weights(cfg, 21)
    folder = U.write_model(str(tmp_path / "m"), cfg, weights)
    eng = Engine.from_folder(folder, dtype="bfloat16", max_slots=n_seqs, max_context=128)
    reqs = [U.random_tokens(30 + i % 7, cfg["vocab_size"], 40 + i) for i in range(n_seqs)]
    outs = U.run_batched(eng, reqs, [14 + i % 5 for i in range(n_seqs)])
    wide = {k: v.double() for k, v in weights.items()}        # (widened once: every request is checked)
    for i in range(n_seqs):
        close("bfloat16")(outs[i], U.plain_logits(cfg, wide, reqs[i]), f"request {i} of {n_seqs}")


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_sizes_that_fit_no_fast_kernel(tmp_path, dtype):
    """Width 100 and inner size 52 (no multiples of 8), heads of 20 (no multiple of 16), an odd
    vocabulary, a window of 1: every matrix-core kernel refuses these, and the engine takes the
    plain kernels instead of giving a wrong result."""
    from agave_amd.engine import Engine
    cfg = dict(P.tiny_config("A"), vocab_size=333, hidden_size=100, num_hidden_layers=3, num_attention_heads=5,
               num_key_value_heads=5, head_dim=20, query_pre_attn_scalar=7, intermediate_size=52,
               sliding_window=1, sliding_window_pattern=3, rms_norm_eps=3e-4)
    cfg.pop("layer_types", None)
    weights = P.random_weights(cfg, 21)
    folder = U.write_model(str(tmp_path / "m"), cfg, weights)
    eng = Engine.from_folder(folder, dtype=dtype, max_slots=3, max_context=160)
    toks = U.random_tokens(130, cfg["vocab_size"], 22)
    ref = U.plain_logits(cfg, weights, toks)
    close(dtype)(U.run_whole(eng, toks), ref, "whole")
    close(dtype)(U.run_tail(eng, toks, 32), ref, "tail")
    outs = U.run_batched(eng, [toks, toks[:70], toks[:9]], (90, 69, 1))
    for o, n in zip(outs, (130, 70, 9)):
        close(dtype)(o, ref[:n], f"batched, {n} tokens")


def test_default_arguments_bound_the_context_and_each_group_s_pool(tmp_path):
    """An engine built with nothing but the folder takes the smaller of the model's context and
    4096 (the reference's default), 0 takes the model's, and each group's storage is as large as
    its reach says: the whole context for layers that need all keys, the window plus a piece for
    the others."""
    from agave_amd.cache import PAGE, pool_pages
    from agave_amd.engine import Engine
    cfg = dict(P.tiny_config("C"), max_position_embeddings=131072)
    folder = U.write_model(str(tmp_path / "m"), cfg, P.random_weights(cfg, 1))
    eng = Engine.from_folder(folder)
    assert eng.max_context == 4096 and eng.max_slots == 8 and eng.dtype == torch.bfloat16
    assert Engine.from_folder(folder, max_context=1000, max_slots=1).max_context == 1000
    del eng
    eng = Engine.from_folder(folder, max_context=0, max_slots=3, prefill_piece=512)
    assert eng.max_context == 131072 and eng.max_piece == 512
    kinds = cfg["layer_types"]
    for key, k_store, v_store, group in zip(eng.cache.group_keys, eng.cache.k_store, eng.cache.v_store, eng.cache.groups):
        n_mem = sum(1 for t in kinds if (t == "sliding_attention") == (key.window is not None))
        want = pool_pages(key.window, 3, 131072, 512)
        assert want == (3 * 2048 if key.window is None else 3 * ((70 + 511 + 62) // 64 + 1))
        assert group.pool.n_pages == want and k_store.shape[:2] == (n_mem, want) and v_store.shape[:2] == (n_mem, want)
    nkv, hd = cfg["num_key_value_heads"], cfg["head_dim"]
    per_page = nkv * PAGE * (64 + hd) * 2            # bfloat16; K rows of 48 are padded to whole tiles of 32 columns
    assert eng.cache.bytes() == per_page * (2 * 3 * 2048 + 3 * 3 * 11)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_through_a_small_window_pool(tmp_path, dtype):
    """One call brings a prompt of 4,200 tokens and a short one while the windowed layers' pool
    holds five pages a sequence: the engine runs the call in pieces, gives pages back between
    them, and returns the wanted rows of all pieces in the caller's order."""
    from agave_amd.engine import Engine
    cfg = dict(P.tiny_config("C"))
    weights = P.random_weights(cfg, 6)
    folder = U.write_model(str(tmp_path / "m"), cfg, weights)
    eng = Engine.from_folder(folder, dtype=dtype, max_slots=2, max_context=4224, prefill_piece=128)
    win = [g for g in eng.cache.groups if g.key.window is not None][0]
    assert win.pool.n_pages == 2 * 5
    long_req = U.random_tokens(4200, cfg["vocab_size"], 9)
    short_req = U.random_tokens(131, cfg["vocab_size"], 10)
    ref_long, ref_short = U.plain_logits(cfg, weights, long_req), U.plain_logits(cfg, weights, short_req)
    want_long = [0, 127, 128, 1000, 1001, 4095, 4096, 4199]
    want_short = [5, 130]
    check = close(dtype)
    kw = dict(longer_sums=8.0) if dtype == "float32" else {}
    slots = [eng.alloc_slot(), eng.alloc_slot()]
    got = eng.step(slots, [long_req, short_req], [want_long, want_short]).float().cpu()
    check(got[:len(want_long)], ref_long[want_long], "long request", **kw)
    check(got[len(want_long):], ref_short[want_short], "short request", **kw)
    assert len(win.held(slots[0])) <= 5 and eng.kv_seq_len(slots[0]) == 4200
    # a call that cannot fit is refused before any piece has run
    from agave_amd.cache import CacheError
    with pytest.raises(CacheError):
        eng.step(slots, [long_req[:200], short_req], "last")
    assert eng.kv_seq_len(slots[0]) == 4200 and eng.kv_seq_len(slots[1]) == 131
    for s in slots:
        eng.free_slot(s)
    # everything wanted in the last piece: the common case of a prompt whose last logits are wanted
    slot = eng.alloc_slot()
    got = eng.step([slot], [long_req[:1000]], "last").float().cpu()
    check(got, ref_long[999:1000], "last row", **kw)
    eng.free_slot(slot)
    for g in eng.cache.groups:
        assert g.pool.n_free == g.pool.n_pages


def test_the_27b_sizes_at_the_whole_context_fit_the_gpu():
    """Gemma 3 27B's own configuration with random weights, 8 slots of 131,072 positions: the
    windowed layers' pool does not grow with the context, so the cache is some 100 GB and the engine
    constructs; a short batch then runs through tables that are 2,048 pages wide."""
    import bench
    from agave_amd.cache import pool_pages
    from agave_amd.engine import Engine
    eng = Engine.from_random(bench.GEMMA3_27B, seed=0, dtype="bfloat16", max_slots=8, max_context=131072)
    page = 2 * 16 * 64 * 128 * 2
    want = page * (10 * pool_pages(None, 8, 131072, 4096) + 52 * pool_pages(1024, 8, 131072, 4096))
    assert eng.cache.bytes() == want and want / 2 ** 30 < 100
    slots = [eng.alloc_slot(), eng.alloc_slot()]
    v = eng.vocab_size
    a = eng.step(slots, [U.random_tokens(70, v, 1), U.random_tokens(3, v, 2)], "last").clone()
    b = eng.step(slots, [[5], [7]], "last").clone()
    assert a.shape == (2, v) and bool(torch.isfinite(a).all()) and bool(torch.isfinite(b).all())
    assert float((a[0] - a[1]).abs().max()) > 0
    for s in slots:
        eng.free_slot(s)
    del eng
    torch.cuda.empty_cache()


@pytest.mark.parametrize("which", ["A", "B", "4b layer"])
def test_bfloat16_against_the_32_bit_path(tmp_path, which):
    """The two paths of one engine on the same folder: how far the bfloat16 logits lie from the 32-bit
    ones, relative to a row's largest logit, and how often both name the same most likely token.
    With random weights many rows have two candidates within rounding of each other, so the rate
    is not 1; where the 32-bit row's winner leads by more than twice the row's error, the
    bfloat16 row must name it too."""
    from agave_amd.engine import Engine
    if which == "4b layer":
        cfg = dict(P.tiny_config("A"), vocab_size=1536, num_hidden_layers=1, sliding_window_pattern=2, rope_theta=1e6,
                   rope_local_base_freq=1e4, rms_norm_eps=1e-6, **BIG_LAYERS["4b"][0])
        cfg.pop("layer_types", None)
        n = 300
    else:
        cfg, n = P.tiny_config(which), 180
    weights = P.random_weights(cfg, 31)
    folder = U.write_model(str(tmp_path / "m"), cfg, weights)
    toks = U.random_tokens(n, cfg["vocab_size"], 32)
    rows = {}
    for dtype in ("float32", "bfloat16"):
        eng = Engine.from_folder(folder, dtype=dtype, max_slots=1, max_context=320)
        rows[dtype] = U.run_tail(eng, toks, 32).double()
        del eng
    f32, bf = rows["float32"], rows["bfloat16"]
    err = (bf - f32).abs().max(-1).values
    rel = err / f32.abs().max(-1).values
    top2 = f32.topk(2, -1).values
    lead = top2[:, 0] - top2[:, 1]
    same = bf.argmax(-1) == f32.argmax(-1)
    rate = float(same.double().mean())
    print(f"{which}: largest relative error {float(rel.max()):.4f}, mean {float(rel.mean()):.4f}, top-1 agreement {rate:.3f}")
    assert float(rel.max()) < 0.04
    assert bool(same[lead > 2 * err].all())
    assert rate >= 0.9
