"""Plain, slow implementation of the Gemma 3 text decoder, used only by tests.

Whole sequences, no cache, one function per part, written from the formulas of
maci0/agave (each function cites the file and lines it was read from).  It
shares no code with ``agave_amd``: it parses ``config.json`` itself, reads the
weights from a plain ``dict`` of HF-named tensors, and does its arithmetic with
ordinary tensor operations on the CPU (float64 by default so that it can serve
as an oracle for the 32-bit engine as well).

Two places follow the build's stated semantics instead of the reference's
behaviour, because the reference never applies them for this architecture:

* the sliding window (a query at position ``p`` sees keys ``max(0, p-W+1)..p``),
  which the reference has in its shared op (``src/ops/attention.zig:92-93``, with
  the callers' convention ``start = sl > W ? sl - W : 0`` at
  ``src/models/gpt_oss.zig:518-519``) but passes ``null`` for in Gemma 3
  (``src/models/gemma3.zig:809-810``);
* ``rope_scaling`` read from the nested HF object (the reference's parser drops
  nested objects, ``src/format/safetensors.zig:1843-1845``); the formula is the
  reference's ``applyRopeScaled`` (``src/models/gemma3.zig:884-902``).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

# --------------------------------------------------------------------------
# configuration (own parse; deliberately independent of agave_amd.config)
# --------------------------------------------------------------------------


def plain_config(cfg: dict) -> dict:
    """Flatten ``text_config`` over the top level (src/format/safetensors.zig:1827-1832)
    and resolve the per-layer kinds (src/models/gemma3.zig:736)."""
    c = dict(cfg)
    if isinstance(cfg.get("text_config"), dict):
        c.update(cfg["text_config"])
    n_layers = int(c["num_hidden_layers"])
    if c.get("layer_types") is not None:
        sliding = [t == "sliding_attention" for t in c["layer_types"]]
    else:
        pattern = int(c.get("sliding_window_pattern", 6))
        # is_local = pattern > 0 and (li + 1) % pattern != 0   (gemma3.zig:736)
        sliding = [pattern > 0 and (i + 1) % pattern != 0 for i in range(n_layers)]
    scaling = c.get("rope_scaling") or {}
    factor = float(scaling.get("factor", 1.0)) if scaling else 1.0
    head_dim = int(c["head_dim"])
    return dict(
        vocab=int(c["vocab_size"]),
        hidden=int(c["hidden_size"]),
        n_layers=n_layers,
        n_heads=int(c["num_attention_heads"]),
        n_kv=int(c["num_key_value_heads"]),
        head_dim=head_dim,
        inter=int(c["intermediate_size"]),
        eps=float(c.get("rms_norm_eps", 1e-6)),
        theta_global=float(c.get("rope_theta", 1e6)),
        theta_local=float(c.get("rope_local_base_freq", 1e4)),
        factor=factor,
        window=int(c["sliding_window"]) if c.get("sliding_window") is not None else None,
        sliding=sliding,
        # scale = 1/sqrt(query_pre_attn_scalar), default head_dim (gemma3.zig:190-194)
        scalar=float(c.get("query_pre_attn_scalar", head_dim)),
    )


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------


def embed(tokens: Sequence[int], table: torch.Tensor, hidden: int) -> torch.Tensor:
    """h = E[token] * sqrt(hidden_size), the scale applied after widening the row
    (src/models/gemma3.zig:195, 1017-1046; research/gemma3_ref.py:253)."""
    idx = torch.as_tensor(list(tokens), dtype=torch.long)
    return table[idx] * math.sqrt(float(hidden))


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float, add_one: bool = True) -> torch.Tensor:
    """y = x * (1/sqrt(mean(x^2) + eps)) * g over the last axis, g = 1 + w for HF
    weights (src/backend/kernels/cpu/norm.zig:7-40; the +1 at
    src/models/gemma3.zig:943-949; research/gemma3_ref.py:157-159)."""
    g = (w + 1.0) if add_one else w
    ms = (x * x).mean(dim=-1, keepdim=True)
    return x * (1.0 / torch.sqrt(ms + eps)) * g


def rope_angles(positions: torch.Tensor, rope_dim: int, theta: float, factor: float = 1.0) -> torch.Tensor:
    """a[p, i] = (pos * 1/factor) * theta^(-2i/rope_dim), i < rope_dim/2
    (src/backend/kernels/cpu/rope.zig:11-48; linear scaling as
    src/models/gemma3.zig:884-902: the position is multiplied by 1/factor)."""
    i = torch.arange(rope_dim // 2, dtype=positions.dtype)
    freq = torch.exp(-math.log(theta) * (2.0 * i) / rope_dim)
    p = positions * (1.0 / factor)
    return p[:, None] * freq[None, :]


def apply_rope(x: torch.Tensor, angles: torch.Tensor) -> torch.Tensor:
    """Split-half rotation of pairs (i, i + half) in every head
    (src/backend/kernels/cpu/rope.zig:11-48; research/kernels/reference.py:30-67):
    x_i' = x_i cos a - x_{i+half} sin a ;  x_{i+half}' = x_i sin a + x_{i+half} cos a.
    x: [T, heads, head_dim]; angles: [T, rope_dim/2]; dims beyond rope_dim are kept."""
    half = angles.shape[-1]
    c = torch.cos(angles)[:, None, :]
    s = torch.sin(angles)[:, None, :]
    re, im, rest = x[..., :half], x[..., half:2 * half], x[..., 2 * half:]
    return torch.cat([re * c - im * s, re * s + im * c, rest], dim=-1)


def softmax_rows(s: torch.Tensor) -> torch.Tensor:
    """max-subtract, exp, sum, multiply by 1/sum (src/backend/kernels/cpu/softmax.zig:7-41)."""
    m = s.max(dim=-1, keepdim=True).values
    e = torch.exp(s - m)
    return e * (1.0 / e.sum(dim=-1, keepdim=True))


def visible(n: int, window: Optional[int]) -> torch.Tensor:
    """Boolean [query, key]: causal, and on sliding layers key >= query - W + 1
    (window convention of src/models/gpt_oss.zig:518-519 with sl = pos + 1)."""
    q = torch.arange(n)[:, None]
    k = torch.arange(n)[None, :]
    ok = k <= q
    if window is not None:
        ok = ok & (k >= q - window + 1)
    return ok


def attention_core(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                   window: Optional[int]) -> torch.Tensor:
    """For query head h, kvh = h / (nh/nkv): s_t = (q_h . k_t) * scale over the visible
    keys, p = softmax(s), o_h = sum_t p_t v_t
    (src/backend/kernels/cpu/sdpa.zig:34-88; tests/sdpa_oracle.zig:133-186).
    q: [T, nh, hd]; k, v: [T, nkv, hd] -> [T, nh, hd]."""
    T, nh, hd = q.shape
    nkv = k.shape[1]
    group = nh // nkv
    ok = visible(T, window)
    out = torch.zeros_like(q)
    for h in range(nh):
        kvh = h // group
        s = (q[:, h, :] @ k[:, kvh, :].T) * scale
        s = s.masked_fill(~ok, float("-inf"))
        out[:, h, :] = softmax_rows(s) @ v[:, kvh, :]
    return out


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """0.5 x (1 + tanh(c (x + 0.044715 x^3))), c = sqrt(2/pi)
    (src/backend/kernels/cpu/activation.zig:69-113; src/ops/math.zig:8-16)."""
    c = 0.7978845608028654
    return 0.5 * x * (1.0 + torch.tanh(c * (x + 0.044715 * x * x * x)))


def geglu(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """f = W_down (gelu_tanh(W_gate x) * (W_up x)) (src/models/gemma3.zig:835-872)."""
    return (gelu_tanh(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


# --------------------------------------------------------------------------
# the block and the whole model
# --------------------------------------------------------------------------

_PREFIXES = ("model.language_model.", "language_model.model.", "model.")  # src/format/safetensors.zig:517-521


def _prefix(weights: Dict[str, torch.Tensor]) -> str:
    for p in _PREFIXES:
        if p + "embed_tokens.weight" in weights:
            return p
    raise KeyError("embed_tokens.weight")


def attention_layer(h: torch.Tensor, w, c: dict, li: int, positions: torch.Tensor) -> torch.Tensor:
    """Pre-norm, q/k/v, per-head q/k norm before rotation, rotation with the layer's
    base, attention, output projection (src/models/gemma3.zig:701-828)."""
    T = h.shape[0]
    nh, nkv, hd = c["n_heads"], c["n_kv"], c["head_dim"]
    x = rms_norm(h, w("input_layernorm.weight"), c["eps"])
    q = (x @ w("self_attn.q_proj.weight").T).view(T, nh, hd)
    k = (x @ w("self_attn.k_proj.weight").T).view(T, nkv, hd)
    v = (x @ w("self_attn.v_proj.weight").T).view(T, nkv, hd)
    q = rms_norm(q, w("self_attn.q_norm.weight"), c["eps"])
    k = rms_norm(k, w("self_attn.k_norm.weight"), c["eps"])
    if c["sliding"][li]:
        ang = rope_angles(positions, hd, c["theta_local"], 1.0)
        window = c["window"]
    else:
        ang = rope_angles(positions, hd, c["theta_global"], c["factor"])
        window = None
    q, k = apply_rope(q, ang), apply_rope(k, ang)
    o = attention_core(q, k, v, 1.0 / math.sqrt(c["scalar"]), window)
    return o.reshape(T, nh * hd) @ w("self_attn.o_proj.weight").T


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: Sequence[int],
            dtype: torch.dtype = torch.float64, first_position: int = 0) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence: embedding, then per layer
    h += post_norm(attention(pre_norm(h))); h += post_norm(ffn(pre_norm(h)))
    (src/models/gemma3.zig:341-348, 823-826, 872-878), final norm, tied or separate
    output matrix (src/models/gemma3.zig:352-359)."""
    c = plain_config(cfg)
    W = {k: v.to(dtype) for k, v in weights.items()}
    p = _prefix(W)
    positions = torch.arange(first_position, first_position + len(tokens), dtype=dtype)
    h = embed(tokens, W[p + "embed_tokens.weight"], c["hidden"])
    for li in range(c["n_layers"]):
        def w(name, li=li):
            return W[f"{p}layers.{li}.{name}"]
        a = attention_layer(h, w, c, li, positions)
        h = h + rms_norm(a, w("post_attention_layernorm.weight"), c["eps"])
        x = rms_norm(h, w("pre_feedforward_layernorm.weight"), c["eps"])
        f = geglu(x, w("mlp.gate_proj.weight"), w("mlp.up_proj.weight"), w("mlp.down_proj.weight"))
        h = h + rms_norm(f, w("post_feedforward_layernorm.weight"), c["eps"])
    h = rms_norm(h, W[p + "norm.weight"], c["eps"])
    head = W["lm_head.weight"] if "lm_head.weight" in W else W[p + "embed_tokens.weight"]
    return h @ head.T


# --------------------------------------------------------------------------
# sampling (host statement of src/ops/math.zig)
# --------------------------------------------------------------------------


def argmax_first(logits: torch.Tensor) -> int:
    """Index of the maximum, first occurrence on ties (src/ops/math.zig:32-50)."""
    m = logits.max()
    return int(torch.nonzero(logits >= m)[0])


def apply_repeat_penalty(logits: torch.Tensor, ids: Sequence[int], penalty: float) -> torch.Tensor:
    """Once for every listed id, repeats included: positive logits are divided by the
    penalty, the others multiplied; ids outside the vocabulary are ignored
    (src/ops/math.zig:186-197)."""
    out = logits.clone()
    for t in ids:
        if 0 <= t < out.numel():
            out[t] = out[t] / penalty if out[t] > 0 else out[t] * penalty
    return out


def sample_distribution(logits: torch.Tensor, temperature: float, top_k: int = 0,
                        top_p: float = 1.0, max_candidates: int = 1024) -> torch.Tensor:
    """The unnormalised weights that src/ops/math.zig:209-362 draws from: logits/T;
    top-k keeps values >= the k-th largest (k capped at 1024, ties kept); exp(x - max);
    top-p sorts the (at most 1024) largest weights, takes the smallest prefix whose mass
    reaches p*sum and keeps every weight >= the last one taken."""
    x = logits.to(torch.float64) / temperature
    n = x.numel()
    if 0 < top_k < n:
        kth = torch.topk(x, min(top_k, max_candidates)).values[-1]
        x = torch.where(x < kth, torch.full_like(x, float("-inf")), x)
    w = torch.exp(x - x.max())
    w = torch.where(torch.isinf(x) & (x < 0), torch.zeros_like(w), w)
    if 0.0 < top_p < 1.0:
        total = w.sum()
        cand = torch.sort(w[w > 0], descending=True).values[:max_candidates]
        cum = torch.cumsum(cand, 0)
        hit = torch.nonzero(cum >= top_p * total)
        threshold = cand[int(hit[0])] if hit.numel() else torch.tensor(0.0, dtype=w.dtype)
        w = torch.where(w < threshold, torch.zeros_like(w), w)
    return w


def sample_token(logits: torch.Tensor, temperature: float, top_k: int, top_p: float, u: float) -> int:
    """temperature 0 -> argmax; else the first index whose running sum of weights
    exceeds u * sum, u in [0, 1) (src/ops/math.zig:210, 365-371)."""
    if temperature == 0:
        return argmax_first(logits)
    w = sample_distribution(logits, temperature, top_k, top_p)
    cum = torch.cumsum(w, 0)
    hit = torch.nonzero(u * w.sum() < cum)
    return int(hit[0]) if hit.numel() else w.numel() - 1


# --------------------------------------------------------------------------
# tiny configurations and random weights for tests (own generator)
# --------------------------------------------------------------------------


def tiny_config(which: str) -> dict:
    """Two tiny configurations that differ in every size and option."""
    if which == "A":
        return dict(
            architectures=["Gemma3ForCausalLM"], model_type="gemma3_text",
            vocab_size=512, hidden_size=64, num_hidden_layers=4, num_attention_heads=4,
            num_key_value_heads=1, head_dim=32, query_pre_attn_scalar=32, intermediate_size=192,
            sliding_window=16, sliding_window_pattern=2, rope_theta=1e6, rope_local_base_freq=1e4,
            rope_scaling=None, rms_norm_eps=1e-6, tie_word_embeddings=True,
            hidden_activation="gelu_pytorch_tanh", max_position_embeddings=4096,
            bos_token_id=2, eos_token_id=1)
    if which == "B":
        return dict(
            architectures=["Gemma3ForCausalLM"], model_type="gemma3_text",
            vocab_size=1000, hidden_size=96, num_hidden_layers=6, num_attention_heads=6,
            num_key_value_heads=2, head_dim=24, query_pre_attn_scalar=16, intermediate_size=320,
            sliding_window=8, sliding_window_pattern=3, rope_theta=5e5, rope_local_base_freq=1e3,
            rope_scaling={"rope_type": "linear", "factor": 8.0}, rms_norm_eps=1e-5,
            tie_word_embeddings=True, hidden_activation="gelu_pytorch_tanh",
            max_position_embeddings=4096, bos_token_id=2, eos_token_id=[1, 106])
    if which == "C":
        # MFMA-sized heads, three KV groups, explicit layer_types, untied head
        return dict(
            architectures=["Gemma3ForCausalLM"], model_type="gemma3_text",
            vocab_size=777, hidden_size=160, num_hidden_layers=5, num_attention_heads=6,
            num_key_value_heads=3, head_dim=48, query_pre_attn_scalar=40, intermediate_size=416,
            sliding_window=70,
            layer_types=["sliding_attention", "full_attention", "sliding_attention",
                         "sliding_attention", "full_attention"],
            rope_theta=2e5, rope_local_base_freq=5e3,
            rope_scaling={"rope_type": "linear", "factor": 4.0}, rms_norm_eps=3e-6,
            tie_word_embeddings=False, hidden_activation="gelu_pytorch_tanh",
            max_position_embeddings=4096, bos_token_id=2, eos_token_id=1)
    raise KeyError(which)


def tensor_shapes(cfg: dict) -> Dict[str, List[int]]:
    c = plain_config(cfg)
    e, qd, kvd, hd, ff = c["hidden"], c["n_heads"] * c["head_dim"], c["n_kv"] * c["head_dim"], c["head_dim"], c["inter"]
    shapes = {"model.embed_tokens.weight": [c["vocab"], e], "model.norm.weight": [e]}
    for i in range(c["n_layers"]):
        p = f"model.layers.{i}."
        shapes.update({
            p + "input_layernorm.weight": [e], p + "self_attn.q_proj.weight": [qd, e],
            p + "self_attn.k_proj.weight": [kvd, e], p + "self_attn.v_proj.weight": [kvd, e],
            p + "self_attn.q_norm.weight": [hd], p + "self_attn.k_norm.weight": [hd],
            p + "self_attn.o_proj.weight": [e, qd], p + "post_attention_layernorm.weight": [e],
            p + "pre_feedforward_layernorm.weight": [e], p + "mlp.gate_proj.weight": [ff, e],
            p + "mlp.up_proj.weight": [ff, e], p + "mlp.down_proj.weight": [e, ff],
            p + "post_feedforward_layernorm.weight": [e]})
    if cfg.get("tie_word_embeddings", True) is False:
        shapes["lm_head.weight"] = [c["vocab"], e]
    return shapes


def random_weights(cfg: dict, seed: int, std: float = 0.02, norm_std: float = 0.1,
                   bf16_exact: bool = True) -> Dict[str, torch.Tensor]:
    """Linear and embedding weights N(0, std), norm weights N(0, norm_std) (used as 1 + w).
    With ``bf16_exact`` every value is representable in bfloat16, so that a 32-bit and a
    bfloat16 engine read the same numbers."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        s = norm_std if len(shape) == 1 else std
        t = torch.randn(shape, generator=g, dtype=torch.float32) * s
        out[name] = t.to(torch.bfloat16).to(torch.float32) if bf16_exact else t
    return out
