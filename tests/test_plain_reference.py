"""Pins the plain implementation by what fixes it beside the reference's text:
vectors the reference's own tests and golden files hold, special cases that reduce
to a library routine, and invariants.  Each case is chosen so that a plausible
mistake (a wrong sign or pairing, a norm in the wrong place) fails it."""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_gemma3 as P

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
needs_golden = pytest.mark.skipif(not os.path.isdir(GOLDEN), reason="reference golden vectors not mounted")


def _g(name):
    return torch.from_numpy(np.fromfile(os.path.join(GOLDEN, name + ".bin"), dtype="<f4").astype(np.float64))


# ---------------------------------------------------------------- RMSNorm

def test_rmsnorm_reference_vector():
    # src/backend/kernels/cpu/norm.zig:135-147: x = 1..8, w = 1 -> x / sqrt(25.5)
    x = torch.arange(1, 9, dtype=torch.float64)
    y = P.rms_norm(x, torch.ones(8, dtype=torch.float64), 0.0, add_one=False)
    assert torch.allclose(y, x / math.sqrt(25.5), atol=1e-12)


def test_rmsnorm_unit_rms_and_scale_invariance():
    x = torch.randn(5, 96, dtype=torch.float64)
    y = P.rms_norm(x, torch.zeros(96, dtype=torch.float64), 1e-12)       # w = 0 -> gain 1
    assert torch.allclose((y * y).mean(-1), torch.ones(5, dtype=torch.float64), atol=1e-9)
    assert torch.allclose(P.rms_norm(7.0 * x, torch.zeros(96, dtype=torch.float64), 1e-12), y, atol=1e-9)
    # eps dominates a tiny input (norm.zig: eps case)
    tiny = torch.full((4,), 1e-20, dtype=torch.float64)
    out = P.rms_norm(tiny, torch.zeros(4, dtype=torch.float64), 1e-6)
    assert torch.allclose(out, tiny / math.sqrt(1e-6), rtol=1e-9, atol=0)


@needs_golden
@pytest.mark.parametrize("n", [128, 1152, 2560, 3136])
def test_rmsnorm_golden(n):
    # research/kernels/generate_golden.py:98-110: eps 1e-5, plain weight
    y = P.rms_norm(_g(f"rms_norm_n{n}_x"), _g(f"rms_norm_n{n}_w"), 1e-5, add_one=False)
    assert torch.allclose(y, _g(f"rms_norm_n{n}_out"), atol=2e-5, rtol=1e-5)


# ---------------------------------------------------------------- RoPE

def test_rope_reference_vector_and_identity():
    # src/backend/kernels/cpu/rope.zig:71-84: [1,0,0,0], pos 1, theta 1e4, dim 4 -> [cos1, 0, sin1, 0]
    x = torch.tensor([1.0, 0, 0, 0], dtype=torch.float64).view(1, 1, 4)
    ang = P.rope_angles(torch.tensor([1.0], dtype=torch.float64), 4, 1e4)
    y = P.apply_rope(x, ang).flatten()
    assert torch.allclose(y, torch.tensor([math.cos(1), 0, math.sin(1), 0], dtype=torch.float64), atol=1e-12)
    x = torch.randn(1, 3, 8, dtype=torch.float64)
    assert torch.equal(P.apply_rope(x, P.rope_angles(torch.zeros(1, dtype=torch.float64), 8, 1e4)), x)


def test_rope_pairing_norms_and_partial_rotation():
    x = torch.randn(4, 2, 12, dtype=torch.float64)
    ang = P.rope_angles(torch.arange(4, dtype=torch.float64), 8, 1e3)    # rope_dim 8 < head_dim 12
    y = P.apply_rope(x, ang)
    assert torch.equal(y[..., 8:], x[..., 8:])                            # tail untouched (rope.zig:96-110)
    # pair (i, i + half) keeps its norm; the interleaved pairing (2i, 2i+1) would not
    assert torch.allclose(y[..., :4] ** 2 + y[..., 4:8] ** 2, x[..., :4] ** 2 + x[..., 4:8] ** 2, atol=1e-12)


def test_rope_relative_property_and_linear_scaling():
    hd = 16
    q = torch.randn(1, 1, hd, dtype=torch.float64)
    k = torch.randn(1, 1, hd, dtype=torch.float64)

    def dot(pq, pk, factor=1.0):
        a = P.apply_rope(q, P.rope_angles(torch.tensor([float(pq)], dtype=torch.float64), hd, 1e4, factor))
        b = P.apply_rope(k, P.rope_angles(torch.tensor([float(pk)], dtype=torch.float64), hd, 1e4, factor))
        return float((a * b).sum())
    assert abs(dot(9, 4) - dot(105, 100)) < 1e-9                          # only the distance counts
    assert abs(dot(9, 4) - dot(4, 9)) > 1e-3                              # and its sign
    # factor 8 at position 8 is the unscaled rotation at position 1
    a = P.rope_angles(torch.tensor([8.0], dtype=torch.float64), hd, 1e4, 8.0)
    b = P.rope_angles(torch.tensor([1.0], dtype=torch.float64), hd, 1e4, 1.0)
    assert torch.allclose(a, b, atol=1e-12)


@needs_golden
@pytest.mark.parametrize("pos", [0, 1, 10, 100, 1000])
def test_rope_golden(pos):
    # research/kernels/generate_golden.py:140-155: nh 4, hd 256, theta 1e4
    for t in ("q", "k"):
        x = _g(f"rope_nh4_hd256_pos{pos}_{t}_in").view(1, 4, 256)
        ang = P.rope_angles(torch.tensor([float(pos)], dtype=torch.float64), 256, 1e4)
        y = P.apply_rope(x, ang).flatten()
        assert torch.allclose(y, _g(f"rope_nh4_hd256_pos{pos}_{t}_out"), atol=2e-4)


# ---------------------------------------------------------------- softmax / attention

def test_softmax_vectors():
    # src/backend/kernels/cpu/softmax.zig:52-67, 104-121, 148-155
    s = P.softmax_rows(torch.tensor([[0.0, math.log(2.0)]], dtype=torch.float64))
    assert torch.allclose(s, torch.tensor([[1 / 3, 2 / 3]], dtype=torch.float64), atol=1e-12)
    s = P.softmax_rows(torch.tensor([[0.0, 0, 0, 1000]], dtype=torch.float64))
    assert torch.isfinite(s).all() and abs(float(s.sum()) - 1) < 1e-12
    s = P.softmax_rows(torch.zeros(1, 7, dtype=torch.float64))
    assert torch.allclose(s, torch.full((1, 7), 1 / 7, dtype=torch.float64))


def test_attention_reduces_to_library_routine():
    # no rotation, no window: softmax(QK^T * scale + causal) V from the library
    T, nh, nkv, hd = 11, 4, 2, 8
    q, k, v = (torch.randn(T, n, hd, dtype=torch.float64) for n in (nh, nkv, nkv))
    out = P.attention_core(q, k, v, 0.3, None)
    kk = k.repeat_interleave(nh // nkv, dim=1)
    vv = v.repeat_interleave(nh // nkv, dim=1)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1),
                                         is_causal=True, scale=0.3).transpose(0, 1)
    assert torch.allclose(out, ref, atol=1e-10)
    # a window at least as long as the sequence changes nothing
    assert torch.allclose(P.attention_core(q, k, v, 0.3, T), out, atol=1e-12)


def test_attention_small_cases():
    # one key -> V; two keys -> [1/(1+e), e/(1+e)] (src/backend/kernels/cpu/sdpa.zig:289-319)
    q = torch.tensor([[[1.0, 0.0]], [[1.0, 0.0]]], dtype=torch.float64)
    k = torch.tensor([[[0.0, 0.0]], [[1.0, 0.0]]], dtype=torch.float64)
    v = torch.tensor([[[1.0, 0.0]], [[0.0, 1.0]]], dtype=torch.float64)
    out = P.attention_core(q, k, v, 1.0, None)
    assert torch.allclose(out[0, 0], v[0, 0])
    e = math.e
    assert torch.allclose(out[1, 0], torch.tensor([1 / (1 + e), e / (1 + e)], dtype=torch.float64), atol=1e-12)
    # heads of one group with equal queries give equal outputs
    T, hd = 6, 4
    q1 = torch.randn(T, 1, hd, dtype=torch.float64).repeat(1, 4, 1)
    k, v = torch.randn(T, 2, hd, dtype=torch.float64), torch.randn(T, 2, hd, dtype=torch.float64)
    o = P.attention_core(q1, k, v, 0.5, None)
    assert torch.allclose(o[:, 0], o[:, 1]) and torch.allclose(o[:, 2], o[:, 3])
    assert not torch.allclose(o[:, 1], o[:, 2])


def test_window_edges():
    # {start=1, len=1} excludes token 0 (src/ops/attention.zig:586-626): W = 1 sees only itself
    T, hd = 5, 4
    q, k, v = (torch.randn(T, 1, hd, dtype=torch.float64) for _ in range(3))
    assert torch.allclose(P.attention_core(q, k, v, 1.0, 1), v, atol=1e-12)
    # W keys including the query's own: key p-W+1 counts, key p-W does not
    W = 3
    base = P.attention_core(q, k, v, 1.0, W)
    k2, v2 = k.clone(), v.clone()
    k2[1] += 5.0; v2[1] += 5.0          # distance W from query 4: outside
    assert torch.allclose(P.attention_core(q, k2, v2, 1.0, W)[4], base[4], atol=1e-12)
    k3, v3 = k.clone(), v.clone()
    k3[2] += 5.0; v3[2] += 5.0          # distance W-1 from query 4: inside
    assert not torch.allclose(P.attention_core(q, k3, v3, 1.0, W)[4], base[4], atol=1e-6)


@needs_golden
@pytest.mark.parametrize("nh,nkv,hd,sl,suffix", [
    (4, 1, 256, 1, "_naive"), (4, 1, 256, 8, "_naive"), (4, 1, 256, 64, "_online"), (4, 1, 256, 256, "_naive"),
    (20, 5, 128, 1, ""), (20, 5, 128, 32, "")])
def test_attention_golden(nh, nkv, hd, sl, suffix):
    # research/kernels/generate_golden.py:56-95: one query over sl keys, scale 1/sqrt(hd)
    tag = f"sdpa_nh{nh}_nkv{nkv}_hd{hd}_sl{sl}"
    q = _g(tag + "_q").view(1, nh, hd)
    keys = _g(tag + "_keys").view(sl, nkv, hd)
    values = _g(tag + "_values").view(sl, nkv, hd)
    # put the query last so that causal attention sees all sl keys
    qq = torch.zeros(sl, nh, hd, dtype=torch.float64)
    qq[-1] = q[0]
    out = P.attention_core(qq, keys, values, 1.0 / math.sqrt(hd), None)[-1].flatten()
    assert torch.allclose(out, _g(tag + "_out" + suffix), atol=2e-5)


# ---------------------------------------------------------------- GeGLU

def test_gelu_values_and_library():
    # src/backend/kernels/cpu/activation.zig:209-215
    x = torch.tensor([0.0, 1.0, -1.0, 2.0, 3.0], dtype=torch.float64)
    want = torch.tensor([0.0, 0.8412, -0.1588, 1.9546, 2.9960], dtype=torch.float64)
    assert torch.allclose(P.gelu_tanh(x), want, atol=1e-3)
    x = torch.randn(1000, dtype=torch.float64) * 3
    assert torch.allclose(P.gelu_tanh(x), F.gelu(x, approximate="tanh"), atol=1e-12)
    assert torch.isfinite(P.gelu_tanh(torch.tensor([-100.0, 100.0], dtype=torch.float64))).all()


@needs_golden
@pytest.mark.parametrize("n", [128, 1152, 6912])
def test_gelu_golden(n):
    assert torch.allclose(P.gelu_tanh(_g(f"gelu_n{n}_x")), _g(f"gelu_n{n}_out"), atol=1e-6)


def test_geglu_is_gelu_then_mul_one_unit():
    x = torch.randn(3, 5, dtype=torch.float64)
    wg, wu, wd = torch.randn(1, 5, dtype=torch.float64), torch.randn(1, 5, dtype=torch.float64), torch.randn(4, 1, dtype=torch.float64)
    ref = (F.gelu(x @ wg.T, approximate="tanh") * (x @ wu.T)) @ wd.T
    assert torch.allclose(P.geglu(x, wg, wu, wd), ref, atol=1e-12)
    # the activation is on the gate, not on the up branch
    assert not torch.allclose(P.geglu(x, wu, wg, wd), ref, atol=1e-6)


# ---------------------------------------------------------------- whole model

def _model(which, seed):
    cfg = P.tiny_config(which)
    return cfg, P.random_weights(cfg, seed)


def test_zero_layer_model_is_embedding_and_tied_head():
    cfg, w = _model("A", 0)
    cfg = dict(cfg, num_hidden_layers=0)
    w = {k: v for k, v in w.items() if ".layers." not in k}
    toks = [3, 77, 500]
    E = w["model.embed_tokens.weight"].double()
    h = E[toks] * math.sqrt(64)
    ref = P.rms_norm(h, w["model.norm.weight"].double(), 1e-6) @ E.T
    assert torch.allclose(P.forward(cfg, w, toks), ref, atol=1e-12)


def test_post_norm_gain_minus_one_switches_branch_off():
    cfg, w = _model("A", 0)
    toks = list(range(20, 40))
    for i in range(cfg["num_hidden_layers"]):
        w[f"model.layers.{i}.post_attention_layernorm.weight"].fill_(-1.0)
        w[f"model.layers.{i}.post_feedforward_layernorm.weight"].fill_(-1.0)
    zero = dict(cfg, num_hidden_layers=0)
    assert torch.allclose(P.forward(cfg, w, toks), P.forward(zero, w, toks), atol=1e-12)


def test_sliding_only_model_forgets_beyond_window():
    cfg, w = _model("A", 0)
    cfg = dict(cfg, sliding_window_pattern=0, layer_types=["sliding_attention"] * 4, sliding_window=5, num_hidden_layers=1)
    toks = [int(t) for t in torch.randint(0, 512, (12,), generator=torch.Generator().manual_seed(3))]
    base = P.forward(cfg, w, toks)[-1]
    far = list(toks); far[11 - 5] = (far[11 - 5] + 1) % 512        # distance W: not seen by one layer
    near = list(toks); near[11 - 4] = (near[11 - 4] + 1) % 512     # distance W-1: seen
    assert torch.allclose(P.forward(cfg, w, far)[-1], base, atol=1e-12)
    assert not torch.allclose(P.forward(cfg, w, near)[-1], base, atol=1e-9)


def test_query_pre_attn_scalar_matters():
    cfg, w = _model("B", 1)
    toks = list(range(5, 25))
    a = P.forward(cfg, w, toks)
    b = P.forward(dict(cfg, query_pre_attn_scalar=cfg["head_dim"]), w, toks)
    assert (a - b).abs().max() > 1e-6


def test_position_shift_invariance_without_scaling_difference():
    # all layers rotate; logits of a model depend on distances only, so shifting every
    # position by the same amount changes nothing (up to rounding)
    cfg, w = _model("B", 1)
    toks = list(range(100, 130))
    a = P.forward(cfg, w, toks)
    b = P.forward(cfg, w, toks, first_position=37)
    assert torch.allclose(a, b, atol=1e-9)


def test_layer_kinds():
    a = P.plain_config(P.tiny_config("A"))["sliding"]
    b = P.plain_config(P.tiny_config("B"))["sliding"]
    assert a == [True, False, True, False]                     # layers 1, 3 global
    assert b == [True, True, False, True, True, False]         # layers 2, 5 global


# ---------------------------------------------------------------- sampling

def test_sampling_rules():
    # src/ops/math.zig:376-384, 474-583, 665-691
    assert P.argmax_first(torch.tensor([1.0, 5.0, 5.0, 2.0])) == 1
    assert P.argmax_first(torch.tensor([float("-inf"), float("-inf")])) == 0
    lg = torch.tensor([0.1, 3.0, 2.5, -1.0, 0.0])
    assert P.sample_token(lg, 0.0, 0, 1.0, 0.99) == 1
    for u in np.linspace(0, 0.999, 50):
        assert P.sample_token(lg, 1.0, 2, 1.0, float(u)) in (1, 2)
    big = torch.tensor([10.0, 0.0, 0.0, 0.0])
    for u in np.linspace(0, 0.999, 20):
        assert P.sample_token(big, 1.0, 0, 0.5, float(u)) == 0
    pen = P.apply_repeat_penalty(torch.tensor([2.0, -2.0, 1.0]), [0, 1, 7, 0], 2.0)
    assert torch.allclose(pen, torch.tensor([0.5, -4.0, 1.0]))
    # frequencies follow softmax(logits / T)
    w = P.sample_distribution(lg, 0.7)
    assert torch.allclose(w / w.sum(), torch.softmax(lg.double() / 0.7, 0), atol=1e-12)
