"""Parts that the framework does not have, defined here and registered from outside: a mixer
with state of its own, a feed-forward with routing, another position encoding, and an
architecture that arranges them with the built-in attention in a run order that names a
layer twice and lets a layer read another layer's cache.  No file of the framework changes:
the model is built from its folder by ``Engine.from_folder`` and stepped like any other.

The toy parts compute with torch on the GPU (they are test fixtures, not product code); the
framework's own parts beside them run their kernels.  Everything is compared with a plain
whole-sequence statement of the same model below.
"""
import json
import math
import os
from dataclasses import dataclass
from typing import List, Optional

import pytest
import torch

import engine_utils as U
import plain_gemma3 as P

pytestmark = pytest.mark.gpu

HIDDEN, VOCAB, HEADS, KV, HD, INTER, EXPERTS, WINDOW = 96, 211, 4, 2, 32, 120, 3, 20
EPS, THETA = 1e-5, 5000.0


# ---------------------------------------------------------------- the toy parts
def define_and_register():
    from agave_amd.cache import StateNeed
    from agave_amd.config import register_architecture
    from agave_amd.config.registry import Architecture
    from agave_amd.config.spec import (AttentionSpec, FeedForwardSpec, GatedFfnSpec, LayerSpec, MixerSpec, ModelSpec,
                                       NormSpec, PositionSpec, RunEntry)
    from agave_amd.parts import register
    from agave_amd.weights.loader import TensorNeed

    @dataclass(frozen=True)
    class DecaySpec(MixerSpec):
        hidden: int = 0
        decay: str = ""
        out_proj: str = ""

    class DecayMixer:
        """s_t = sigmoid(d) * s_{t-1} + x_t ;  y_t = W s_t.  The state s is kept per sequence.
        It says that it takes the normalised rows as a promise (a step of one row hands it a
        ``NormedRows``) and asks for the tensor itself, as a part from outside may."""
        takes_rows_to_be_normed = True

        def __init__(self, spec, weights, env):
            self.a = torch.sigmoid(weights.get(spec.decay).float().to(env.device))
            self.w = weights.get(spec.out_proj).float().to(env.device)
            self.spec, self.env = spec, env

        @staticmethod
        def tensor_needs(spec):
            return [TensorNeed(spec.decay, (spec.hidden,)), TensorNeed(spec.out_proj, (spec.hidden, spec.hidden))]

        def kv_need(self):
            return None

        def state_need(self):
            return StateNeed((self.spec.hidden,), torch.float32)

        def forward(self, x, step, memory, writes=True):
            from agave_amd.parts import NormedRows
            if isinstance(x, NormedRows):
                assert x.shape[0] == 1 and not x.taken
                x = x.rows()
            state = step.cache.state[memory]
            xf = x.float()
            if step.is_decode:                       # device indices only: the step may be a graph replay
                idx = step.slots_dev.long()
                s = self.a * state[idx] + xf
                state[idx] = s
                return (s @ self.w.T).to(x.dtype)
            out = torch.empty_like(xf)
            for i, slot in enumerate(step.slots):
                s = state[slot].clone()
                for t in range(step.cu[i], step.cu[i + 1]):
                    s = self.a * s + xf[t]
                    out[t] = s
                state[slot] = s
            return (out @ self.w.T).to(x.dtype)

    @dataclass(frozen=True)
    class TopOneSpec(FeedForwardSpec):
        hidden: int = 0
        intermediate: int = 0
        experts: int = 0
        router: str = ""
        w_in: str = ""
        w_out: str = ""

    class TopOneFfn:
        """Router logits in 32-bit; the token goes through the one expert with the largest logit,
        weighted by how far its softmax weight lies above the second largest (so the output is
        continuous where the choice changes, and rounding cannot make a large difference)."""

        def __init__(self, spec, weights, env):
            self.r = weights.get(spec.router).float().to(env.device)
            self.w_in = weights.get(spec.w_in).float().to(env.device)
            self.w_out = weights.get(spec.w_out).float().to(env.device)

        @staticmethod
        def tensor_needs(spec):
            return [TensorNeed(spec.router, (spec.experts, spec.hidden)),
                    TensorNeed(spec.w_in, (spec.experts, spec.intermediate, spec.hidden)),
                    TensorNeed(spec.w_out, (spec.experts, spec.hidden, spec.intermediate))]

        def forward(self, x, step):
            xf = x.float()
            logits = xf @ self.r.T
            p = torch.softmax(logits, -1)
            e = logits.argmax(-1)
            hid = torch.nn.functional.gelu(torch.einsum("eih,nh->nei", self.w_in, xf), approximate="tanh")
            y = torch.einsum("ehi,nei->neh", self.w_out, hid)
            top2 = p.topk(2, -1).values
            pick = torch.nn.functional.one_hot(e, logits.shape[-1]).float() * (top2[:, :1] - top2[:, 1:])
            return torch.einsum("neh,ne->nh", y, pick).to(x.dtype)

    class WobblePosition:
        """Not a rotation: every element of q and k is multiplied by 1 + 0.3 cos(pos * f_i)."""

        def __init__(self, spec, env):
            i = torch.arange(spec.rotary_dim, dtype=torch.float32, device=env.device)
            self.f = 0.05 + 0.01 * i

        def apply(self, q, k, step):
            pos = step.tok_pos.float()[:, None]
            m = 1.0 + 0.3 * torch.cos(pos * self.f[None, :])          # [N, head_dim]
            for t in (q, k):
                if t is not None:
                    n = t.shape[0]
                    v = t.view(n, -1, m.shape[1]) if t.is_contiguous() else t.reshape(n, -1, m.shape[1])
                    t.copy_((v.float() * m[:, None, :]).to(t.dtype).reshape(n, -1))

    register("mixer", "toy_decay", DecayMixer)
    register("ffn", "toy_top_one", TopOneFfn)
    register("position", "toy_wobble", WobblePosition)

    def norm(name):
        return NormSpec("rmsnorm", HIDDEN, EPS, name, True)

    def attention(prefix, window, position):
        return AttentionSpec(kind="attention", hidden=HIDDEN, n_heads=HEADS, n_kv_heads=KV, head_dim=HD,
                             scale=1.0 / math.sqrt(HD), window=window, position=position,
                             q_norm=NormSpec("rmsnorm", HD, EPS, prefix + "qn", True),
                             k_norm=NormSpec("rmsnorm", HD, EPS, prefix + "kn", True),
                             q_proj=prefix + "q", k_proj=prefix + "k", v_proj=prefix + "v", o_proj=prefix + "o")

    def dense(prefix):
        return GatedFfnSpec(kind="gated_dense", hidden=HIDDEN, intermediate=INTER, activation="gelu_tanh",
                            gate_proj=prefix + "g", up_proj=prefix + "u", down_proj=prefix + "d")

    def layer(i, kind, mixer, ffn):
        return LayerSpec(kind=kind, mixer=mixer, ffn=ffn, pre_mixer_norm=norm(f"l{i}.n0"),
                         post_mixer_norm=norm(f"l{i}.n1"), pre_ffn_norm=norm(f"l{i}.n2"),
                         post_ffn_norm=norm(f"l{i}.n3"))

    def spec_of(cfg, names=None):
        rope = PositionSpec("rope", HD, THETA, 1.0)
        layers = [
            layer(0, "prenorm", DecaySpec("toy_decay", HIDDEN, "l0.decay", "l0.w"),
                  TopOneSpec("toy_top_one", HIDDEN, INTER, EXPERTS, "l0.router", "l0.w_in", "l0.w_out")),
            layer(1, "sandwich", attention("l1.", WINDOW, PositionSpec("toy_wobble", HD)), dense("l1.")),
            layer(2, "sandwich", attention("l2.", None, rope), dense("l2.")),
            layer(3, "sandwich", attention("l3.", None, rope), dense("l3.")),
        ]
        order = [RunEntry(0, 0), RunEntry(1, 1), RunEntry(2, 2),
                 RunEntry(0, 3),                       # layer 0 again, with a state of its own
                 RunEntry(3, 2, writes=False)]         # layer 3 reads what layer 2 cached and appends nothing
        return ModelSpec(architecture="ToyMixForCausalLM", vocab_size=VOCAB, hidden=HIDDEN, embed_weight="emb",
                         embed_scale=1.0, layers=layers, order=order, final_norm=norm("final"), head_weight="head",
                         max_context=cfg["max_position_embeddings"], eos_token_ids=())

    register_architecture(Architecture("ToyMixForCausalLM", ("toy_mix",), lambda raw: dict(raw), spec_of))
    return spec_of


def toy_weights(seed):
    from agave_amd.engine.model import tensor_needs
    spec = define_and_register()({"max_position_embeddings": 512})
    g = torch.Generator().manual_seed(seed)
    out = {}
    for need in tensor_needs(spec):
        std = 0.1 if len(need.shape) > 1 else 0.3
        out[need.name] = (torch.randn(need.shape, generator=g) * std).bfloat16().float()
    out["emb"] = (out["emb"] * 10).bfloat16().float()
    return spec, out


# ---------------------------------------------------------------- the same model, plainly
def plain_toy(w, tokens) -> torch.Tensor:
    W = {k: v.double() for k, v in w.items()}
    T = len(tokens)
    pos = torch.arange(T, dtype=torch.float64)
    h = W["emb"][torch.tensor(tokens)]

    def n(x, name):
        return P.rms_norm(x, W[name], EPS)

    def decay(x):
        a = torch.sigmoid(W["l0.decay"])
        s = torch.zeros(HIDDEN, dtype=torch.float64)
        out = []
        for t in range(T):
            s = a * s + x[t]
            out.append(s)
        return torch.stack(out) @ W["l0.w"].T

    def top_one(x):
        logits = x @ W["l0.router"].T
        p = P.softmax_rows(logits)
        out = torch.zeros_like(x)
        for t in range(T):
            e = int(logits[t].argmax())
            second = max(float(p[t, j]) for j in range(EXPERTS) if j != e)
            out[t] = (p[t, e] - second) * (W["l0.w_out"][e] @ P.gelu_tanh(W["l0.w_in"][e] @ x[t]))
        return out

    def qkv(pre, x, position):
        q = n_heads(x @ W[pre + "q"].T, HEADS, pre + "qn")
        k = n_heads(x @ W[pre + "k"].T, KV, pre + "kn")
        v = (x @ W[pre + "v"].T).view(T, KV, HD)
        if position == "rope":
            ang = P.rope_angles(pos, HD, THETA, 1.0)
            q, k = P.apply_rope(q, ang), P.apply_rope(k, ang)
        else:
            m = 1.0 + 0.3 * torch.cos(pos[:, None] * (0.05 + 0.01 * torch.arange(HD, dtype=torch.float64))[None, :])
            q, k = q * m[:, None, :], k * m[:, None, :]
        return q, k, v

    def n_heads(x, heads, gain):
        return P.rms_norm(x.view(T, heads, HD), W[gain], EPS)

    def ffn(pre, x):
        return P.geglu(x, W[pre + "g"], W[pre + "u"], W[pre + "d"])

    scale = 1.0 / math.sqrt(HD)
    # layer 0 (prenorm: a norm after the routed feed-forward would blow up the small outputs near a
    # change of expert and make the model discontinuous there): decay mixer, routed feed-forward
    h = h + decay(n(h, "l0.n0"))
    h = h + top_one(n(h, "l0.n2"))
    # layer 1 (sandwich): windowed attention with the wobble
    q, k, v = qkv("l1.", n(h, "l1.n0"), "wobble")
    h = h + n(P.attention_core(q, k, v, scale, WINDOW).reshape(T, -1) @ W["l1.o"].T, "l1.n1")
    h = h + n(ffn("l1.", n(h, "l1.n2")), "l1.n3")
    # layer 2 (sandwich): global attention; its keys and values are read again below
    q, k2, v2 = qkv("l2.", n(h, "l2.n0"), "rope")
    h = h + n(P.attention_core(q, k2, v2, scale, None).reshape(T, -1) @ W["l2.o"].T, "l2.n1")
    h = h + n(ffn("l2.", n(h, "l2.n2")), "l2.n3")
    # layer 0 once more, its state starting from zero again
    h = h + decay(n(h, "l0.n0"))
    h = h + top_one(n(h, "l0.n2"))
    # layer 3: its own queries over layer 2's keys and values
    q, _, _ = qkv("l3.", n(h, "l3.n0"), "rope")
    h = h + n(P.attention_core(q, k2, v2, scale, None).reshape(T, -1) @ W["l3.o"].T, "l3.n1")
    h = h + n(ffn("l3.", n(h, "l3.n2")), "l3.n3")
    return n(h, "final") @ W["head"].T


# ---------------------------------------------------------------- the tests
@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    from safetensors.torch import save_file
    spec, w = toy_weights(5)
    folder = str(tmp_path_factory.mktemp("toy"))
    save_file({k: v.bfloat16().contiguous() for k, v in w.items()}, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump({"architectures": ["ToyMixForCausalLM"], "model_type": "toy_mix", "max_position_embeddings": 512}, f)
    return folder, w


def close(got, ref, dtype, what):
    scale = float(ref.abs().max())
    err = (got.double() - ref).abs().max(dim=-1).values
    tol = 3e-5 if dtype == "float32" else 0.04
    assert float(err.max()) <= tol * scale, f"{what}: error {float(err.max()):.3e} of {scale:.3e} at row {int(err.argmax())}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_model_is_built_and_stepped(toy, dtype):
    from agave_amd.engine import Engine
    folder, w = toy
    eng = Engine.from_folder(folder, dtype=dtype, max_slots=3, max_context=256)
    assert set(eng.cache.state) == {0, 3}                       # the decay mixer's two runs, a state each
    assert sorted(eng.cache.group_of_memory) == [1, 2]          # the two attention memories; layer 3 has none
    assert len(eng.cache.groups) == 2                           # a window group and a group of all keys
    assert not eng._prompt_graphs_ok                            # a mixer that does not say so is never recorded over a prompt

    toks = U.random_tokens(100, VOCAB, 1)
    ref = plain_toy(w, toks)
    close(U.run_whole(eng, toks), ref, dtype, "whole")
    close(U.run_tail(eng, toks, 32), ref, dtype, "last 32 one by one (graph replays among them)")

    # batches of unequal lengths, one after another: slots, pages and states are used again
    for b, (lens, first) in enumerate([((50, 21, 80), (30, 21, 2)), ((70, 33), (69, 1)), ((90, 9, 40), (5, 9, 38))]):
        reqs = [U.random_tokens(n, VOCAB, 10 * b + i) for i, n in enumerate(lens)]
        outs = U.run_batched(eng, reqs, first)
        for i, (r, o) in enumerate(zip(reqs, outs)):
            close(o, plain_toy(w, r), dtype, f"batch {b} request {i}")
    assert eng.cache.slots.n_free == eng.cache.max_slots


def test_toy_model_generates(toy):
    """Greedy generation through the entry point, against the plain model's own greedy loop."""
    from agave_amd.engine import Engine
    from agave_amd.sampling import SamplingParams
    folder, w = toy
    eng = Engine.from_folder(folder, dtype="float32", max_slots=2, max_context=128)
    prompts = [U.random_tokens(7, VOCAB, 50), U.random_tokens(19, VOCAB, 51)]
    res = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=6))
    for p, r in zip(prompts, res):
        seq = list(p)
        for _ in range(6):
            seq.append(P.argmax_first(plain_toy(w, seq)[-1]))
        assert list(r.tokens) == seq[len(p):]


# ---------------------------------------------------------------- another kind of norm, and no final norm
def define_centred_norm_model():
    """A norm that subtracts the mean and has a bias, registered from outside, standing before and
    after sublayers next to the built-in RMS norm, in a model with or without a final norm."""
    from agave_amd.config import register_architecture
    from agave_amd.config.registry import Architecture
    from agave_amd.config.spec import AttentionSpec, GatedFfnSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec, RunEntry
    from agave_amd.parts import Norm, register
    from agave_amd.weights.loader import TensorNeed

    class CentredNorm(Norm):
        """y = (x - mean(x)) / sqrt(var(x) + eps) * g + b"""

        def __init__(self, spec, weights, env):
            self.g = weights.get(spec.weight).float().to(env.device)
            self.b = weights.get(spec.weight + "_bias").float().to(env.device)
            self.eps, self.size = spec.eps, spec.size

        @staticmethod
        def tensor_needs(spec):
            return [TensorNeed(spec.weight, (spec.size,)), TensorNeed(spec.weight + "_bias", (spec.size,))]

        def _norm(self, x):
            x = x.float()
            x = x - x.mean(-1, keepdim=True)
            return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + self.eps) * self.g + self.b

        def apply(self, x, out, rows=None):
            out.copy_(self._norm(x if rows is None else x[rows.long()]).to(out.dtype))

        def add_to(self, h, branch):
            h += self._norm(branch.sum(0) if branch.dim() == 3 else branch)

    register("norm", "toy_centred", CentredNorm)

    def rms(name):
        return NormSpec("rmsnorm", HIDDEN, EPS, name, True)

    def centred(name):
        return NormSpec("toy_centred", HIDDEN, EPS, name)

    def attention(prefix):
        return AttentionSpec(kind="attention", hidden=HIDDEN, n_heads=HEADS, n_kv_heads=KV, head_dim=HD,
                             scale=1.0 / math.sqrt(HD), window=None, position=PositionSpec("rope", HD, THETA, 1.0),
                             q_proj=prefix + "q", k_proj=prefix + "k", v_proj=prefix + "v", o_proj=prefix + "o")

    def dense(prefix):
        return GatedFfnSpec(kind="gated_dense", hidden=HIDDEN, intermediate=INTER, activation="gelu_tanh",
                            gate_proj=prefix + "g", up_proj=prefix + "u", down_proj=prefix + "d")

    def spec_of(cfg, names=None):
        layers = [
            LayerSpec("sandwich", attention("l0."), dense("l0."), pre_mixer_norm=rms("l0.n0"),
                      post_mixer_norm=centred("l0.n1"), pre_ffn_norm=centred("l0.n2"), post_ffn_norm=rms("l0.n3")),
            LayerSpec("prenorm", attention("l1."), dense("l1."), pre_mixer_norm=centred("l1.n0"), pre_ffn_norm=rms("l1.n2")),
            LayerSpec("sandwich", attention("l2."), dense("l2."), pre_mixer_norm=rms("l2.n0"),
                      post_mixer_norm=rms("l2.n1"), pre_ffn_norm=rms("l2.n2"), post_ffn_norm=centred("l2.n3")),
        ]
        final = {"none": None, "centred": centred("final"), "rms": rms("final")}[cfg["final_norm"]]
        return ModelSpec(architecture="ToyNormForCausalLM", vocab_size=VOCAB, hidden=HIDDEN, embed_weight="emb",
                         embed_scale=1.0, layers=layers, order=[RunEntry(i, i) for i in range(3)], final_norm=final,
                         head_weight="head", max_context=cfg["max_position_embeddings"], eos_token_ids=())

    register_architecture(Architecture("ToyNormForCausalLM", ("toy_norm",), lambda raw: dict(raw), spec_of))
    return spec_of


def plain_centred_norm_model(w, tokens, final) -> torch.Tensor:
    W = {k: v.double() for k, v in w.items()}
    T = len(tokens)
    ang = P.rope_angles(torch.arange(T, dtype=torch.float64), HD, THETA, 1.0)

    def rms(x, name):
        return P.rms_norm(x, W[name], EPS)

    def centred(x, name):
        x = x - x.mean(-1, keepdim=True)
        return x / torch.sqrt((x * x).mean(-1, keepdim=True) + EPS) * W[name] + W[name + "_bias"]

    def attn(pre, x):
        q = P.apply_rope((x @ W[pre + "q"].T).view(T, HEADS, HD), ang)
        k = P.apply_rope((x @ W[pre + "k"].T).view(T, KV, HD), ang)
        v = (x @ W[pre + "v"].T).view(T, KV, HD)
        return P.attention_core(q, k, v, 1.0 / math.sqrt(HD), None).reshape(T, -1) @ W[pre + "o"].T

    def ffn(pre, x):
        return P.geglu(x, W[pre + "g"], W[pre + "u"], W[pre + "d"])

    h = W["emb"][torch.tensor(tokens)]
    h = h + centred(attn("l0.", rms(h, "l0.n0")), "l0.n1")
    h = h + rms(ffn("l0.", centred(h, "l0.n2")), "l0.n3")
    h = h + attn("l1.", centred(h, "l1.n0"))
    h = h + ffn("l1.", rms(h, "l1.n2"))
    h = h + rms(attn("l2.", rms(h, "l2.n0")), "l2.n1")
    h = h + centred(ffn("l2.", rms(h, "l2.n2")), "l2.n3")
    if final == "centred":
        h = centred(h, "final")
    elif final == "rms":
        h = rms(h, "final")
    return h @ W["head"].T


@pytest.mark.parametrize("final", ["none", "centred", "rms"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_norm_of_another_form_and_a_model_without_a_final_norm(tmp_path, dtype, final):
    """The norm kind is registered here; blocks and the model's end reach every norm through the
    norm part's own interface, so no file of the framework knows of it.  Without a final norm the
    output matrix takes the wanted rows of the residual stream as they are."""
    from safetensors.torch import save_file
    from agave_amd.engine import Engine
    from agave_amd.engine.model import tensor_needs
    cfg = {"architectures": ["ToyNormForCausalLM"], "model_type": "toy_norm", "max_position_embeddings": 256,
           "final_norm": final}
    spec = define_centred_norm_model()(cfg)
    g = torch.Generator().manual_seed(11)
    w = {}
    for need in tensor_needs(spec):
        std = 0.1 if len(need.shape) > 1 else 0.3
        w[need.name] = (torch.randn(need.shape, generator=g) * std).bfloat16().float()
    w["emb"] = (w["emb"] * 10).bfloat16().float()
    assert ("final" in w) == (final != "none") and ("final_bias" in w) == (final == "centred")
    folder = str(tmp_path)
    save_file({k: v.bfloat16().contiguous() for k, v in w.items()}, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    eng = Engine.from_folder(folder, dtype=dtype, max_slots=3, max_context=192)
    assert (eng.model.final_norm is None) == (final == "none")
    toks = U.random_tokens(90, VOCAB, 2)
    ref = plain_centred_norm_model(w, toks, final)
    close(U.run_whole(eng, toks), ref, dtype, "whole")
    close(U.run_tail(eng, toks, 32), ref, dtype, "last 32 one by one")
    slot = eng.alloc_slot()
    some = eng.step([slot], [toks], [[3, 50, 89]]).float().cpu()       # chosen rows only
    eng.free_slot(slot)
    close(some, ref[[3, 50, 89]], dtype, "chosen rows")
    reqs = [U.random_tokens(n, VOCAB, 20 + i) for i, n in enumerate((40, 9, 70))]
    for i, (r, o) in enumerate(zip(reqs, U.run_batched(eng, reqs, (30, 9, 2)))):
        close(o, plain_centred_norm_model(w, r, final), dtype, f"request {i} of a batch")


def test_a_head_norm_that_the_q_k_kernel_cannot_compute_is_refused_by_name():
    """The per-head norm of queries and keys is computed inside the q/k kernel, which knows the
    RMS kind (a gain and an eps): a norm part of another form in that place is refused when the
    mixer is built, with a message that names it, instead of failing at the first step."""
    from agave_amd.config.spec import AttentionSpec, NormSpec, PositionSpec
    from agave_amd.parts import BuildEnv, Workspace, lookup
    from agave_amd.weights.loader import DictWeightSource
    define_centred_norm_model()
    spec = AttentionSpec(kind="attention", hidden=HIDDEN, n_heads=HEADS, n_kv_heads=KV, head_dim=HD, scale=0.25,
                         window=None, position=PositionSpec("rope", HD, THETA, 1.0),
                         q_norm=NormSpec("toy_centred", HD, EPS, "qn"), k_norm=NormSpec("rmsnorm", HD, EPS, "kn"),
                         q_proj="q", k_proj="k", v_proj="v", o_proj="o")
    cls = lookup("mixer", "attention")
    w = {n.name: torch.zeros(n.shape) for n in cls.tensor_needs(spec)}
    env = BuildEnv(torch.float32, torch.device("cuda:0"), Workspace(torch.device("cuda:0")))
    with pytest.raises(ValueError, match="q_norm of kind 'toy_centred'"):
        cls(spec, DictWeightSource(w, cls.tensor_needs(spec)), env)


# ---------------------------------------------------------------- biases on every product, logits scaled and capped
BIAS_INTER, BIAS_WINDOW, LOGIT_SCALE, LOGIT_CAP = 144, 24, 3.0, 2.5


def define_biased_model():
    """The built-in attention and gated feed-forward with a bias on each of their products (and on
    some only), SiLU and the tanh form of GELU as gates, and logits that are multiplied by a factor
    and soft-capped: all of it is the specs' data, no part is defined here."""
    from agave_amd.config import register_architecture
    from agave_amd.config.registry import Architecture
    from agave_amd.config.spec import AttentionSpec, GatedFfnSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec, RunEntry

    def rms(name):
        return NormSpec("rmsnorm", HIDDEN, EPS, name, True)

    def attention(prefix, window, biases):
        names = {f"{p}_bias": prefix + p + "b" for p in biases}
        return AttentionSpec(kind="attention", hidden=HIDDEN, n_heads=HEADS, n_kv_heads=KV, head_dim=HD,
                             scale=1.0 / math.sqrt(HD), window=window, position=PositionSpec("rope", HD, THETA, 1.0),
                             q_proj=prefix + "q", k_proj=prefix + "k", v_proj=prefix + "v", o_proj=prefix + "o", **names)

    def dense(prefix, activation, biases):
        names = {f"{p}_bias": prefix + p[0] + "b" for p in biases}
        return GatedFfnSpec(kind="gated_dense", hidden=HIDDEN, intermediate=BIAS_INTER, activation=activation,
                            gate_proj=prefix + "g", up_proj=prefix + "u", down_proj=prefix + "d", **names)

    def spec_of(cfg, names=None):
        layers = [
            LayerSpec("prenorm", attention("l0.", None, ("q", "k", "v", "o")), dense("l0.", "silu", ("gate", "up", "down")),
                      pre_mixer_norm=rms("l0.n0"), pre_ffn_norm=rms("l0.n2")),
            LayerSpec("prenorm", attention("l1.", BIAS_WINDOW, ("v",)), dense("l1.", "gelu_tanh", ("down",)),
                      pre_mixer_norm=rms("l1.n0"), pre_ffn_norm=rms("l1.n2")),
            LayerSpec("prenorm", attention("l2.", None, ("q", "o")), dense("l2.", "gelu_tanh", ("up",)),
                      pre_mixer_norm=rms("l2.n0"), pre_ffn_norm=rms("l2.n2")),
        ]
        return ModelSpec(architecture="ToyBiasForCausalLM", vocab_size=VOCAB, hidden=HIDDEN, embed_weight="emb",
                         embed_scale=1.0, layers=layers, order=[RunEntry(i, i) for i in range(3)], final_norm=rms("final"),
                         head_weight=None, max_context=cfg["max_position_embeddings"], eos_token_ids=(),
                         logit_scale=cfg["logit_scale"], logit_softcap=cfg["logit_softcap"])

    register_architecture(Architecture("ToyBiasForCausalLM", ("toy_bias",), lambda raw: dict(raw), spec_of))
    return spec_of


def plain_biased_model(w, tokens, scale, cap) -> torch.Tensor:
    W = {k: v.double() for k, v in w.items()}
    T = len(tokens)
    ang = P.rope_angles(torch.arange(T, dtype=torch.float64), HD, THETA, 1.0)

    def b(name):
        return W[name] if name in W else 0.0

    def rms(x, name):
        return P.rms_norm(x, W[name], EPS)

    def attn(pre, x, window):
        q = P.apply_rope((x @ W[pre + "q"].T + b(pre + "qb")).view(T, HEADS, HD), ang)
        k = P.apply_rope((x @ W[pre + "k"].T + b(pre + "kb")).view(T, KV, HD), ang)
        v = (x @ W[pre + "v"].T + b(pre + "vb")).view(T, KV, HD)
        return P.attention_core(q, k, v, 1.0 / math.sqrt(HD), window).reshape(T, -1) @ W[pre + "o"].T + b(pre + "ob")

    def ffn(pre, x, act):
        gate, up = x @ W[pre + "g"].T + b(pre + "gb"), x @ W[pre + "u"].T + b(pre + "ub")
        gate = gate * torch.sigmoid(gate) if act == "silu" else P.gelu_tanh(gate)
        return (gate * up) @ W[pre + "d"].T + b(pre + "db")

    h = W["emb"][torch.tensor(tokens)]
    for pre, window, act in (("l0.", None, "silu"), ("l1.", BIAS_WINDOW, "gelu_tanh"), ("l2.", None, "gelu_tanh")):
        h = h + attn(pre, rms(h, pre + "n0"), window)
        h = h + ffn(pre, rms(h, pre + "n2"), act)
    logits = rms(h, "final") @ W["emb"].T * scale
    return cap * torch.tanh(logits / cap) if cap > 0 else logits


@pytest.mark.parametrize("scale,cap", [(LOGIT_SCALE, LOGIT_CAP), (0.5, 0.0)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_biases_on_the_products_and_logits_scaled_and_capped(tmp_path, dtype, scale, cap):
    """Biases are named by the specs of the attention and of the feed-forward, the logits' factor and
    cap by the model's: a model that has them is stated in data alone.  The biases are drawn as
    large as the products they are added to, and the cap lies inside the logits' range, so that
    leaving one out, or capping before scaling, moves the logits far beyond rounding."""
    from safetensors.torch import save_file
    from agave_amd.engine import Engine
    from agave_amd.engine.model import tensor_needs
    cfg = {"architectures": ["ToyBiasForCausalLM"], "model_type": "toy_bias", "max_position_embeddings": 256,
           "logit_scale": scale, "logit_softcap": cap}
    spec = define_biased_model()(cfg)
    g = torch.Generator().manual_seed(12)
    w = {}
    for need in tensor_needs(spec):
        std = 0.1 if len(need.shape) > 1 else (1.0 if need.name.endswith("b") else 0.3)
        w[need.name] = (torch.randn(need.shape, generator=g) * std).bfloat16().float()
    assert sum(1 for k in w if k.endswith("b") and k != "emb") == 4 + 3 + 1 + 1 + 2 + 1
    folder = str(tmp_path)
    save_file({k: v.bfloat16().contiguous() for k, v in w.items()}, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    eng = Engine.from_folder(folder, dtype=dtype, max_slots=3, max_context=192)
    toks = U.random_tokens(100, VOCAB, 3)
    ref = plain_biased_model(w, toks, scale, cap)
    if cap > 0:
        assert float(ref.abs().max()) > 0.9 * cap and float((ref.abs() < 0.5 * cap).float().mean()) > 0.2, \
            "the cap must bend some logits and leave others"
    # (each bias matters: without it the plain model's logits move by far more than the tolerance)
    for name in [k for k in w if k.endswith("b") and k != "emb"]:
        without = dict(w)
        without[name] = torch.zeros_like(w[name])
        moved = float((plain_biased_model(without, toks, scale, cap) - ref).abs().max())
        assert moved > 0.02 * float(ref.abs().max()), f"{name} would not be missed ({moved:.3e})"     # (the 32-bit run sees 3e-5)
    close(U.run_whole(eng, toks), ref, dtype, "whole")
    close(U.run_tail(eng, toks, 32), ref, dtype, "last 32 one by one")
    reqs = [U.random_tokens(n, VOCAB, 30 + i) for i, n in enumerate((40, 9, 70))]
    for i, (r, o) in enumerate(zip(reqs, U.run_batched(eng, reqs, (30, 9, 2)))):
        close(o, plain_biased_model(w, r, scale, cap), dtype, f"request {i} of a batch")
    # sampling sees the capped logits: greedy generation agrees with the plain model's own loop
    if dtype == "float32":
        from agave_amd.sampling import SamplingParams
        prompt = U.random_tokens(11, VOCAB, 40)
        res = eng.generate([prompt], SamplingParams(temperature=0.0, max_tokens=5))[0]
        seq = list(prompt)
        for _ in range(5):
            seq.append(P.argmax_first(plain_biased_model(w, seq, scale, cap)[-1]))
        assert list(res.tokens) == seq[len(prompt):]
