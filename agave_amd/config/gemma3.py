"""Typed configuration of the Gemma 3 text decoder, read from config.json's own keys.

Reference: the keys the reference reads and their fallbacks are in
``src/models/gemma3.zig:30-55, 149-203`` and ``src/format/safetensors.zig:641-688``;
``text_config`` overrides the top level (``src/format/safetensors.zig:1827-1832``).
Unlike the reference this parser also reads ``vocab_size``, ``sliding_window``,
``layer_types`` and the nested ``rope_scaling`` object, which the reference's
safetensors parser drops (``src/format/safetensors.zig:1843-1845``).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Iterable, List, Optional, Tuple

from .errors import ConfigError
from .spec import (AttentionSpec, GatedFfnSpec, LayerSpec, ModelSpec, NormSpec,
                   PositionSpec, RunEntry)

# Fallbacks of optional keys, as the reference has them (src/models/gemma3.zig:30-55).
# Sizes have no fallback: a missing size is an error that names the key.
_OPTIONAL_DEFAULTS = {
    "rope_theta": 1_000_000.0,          # gemma3.zig:35
    "rope_local_base_freq": 10_000.0,   # gemma3.zig:37
    "rms_norm_eps": 1e-6,               # gemma3.zig:39
    "sliding_window_pattern": 6,        # gemma3.zig:33
    "max_position_embeddings": 4096,    # gemma3.zig:55
}

# Tensor name prefixes tried in this order (src/format/safetensors.zig:517-521).
TENSOR_PREFIXES = ("model.language_model.", "language_model.model.", "model.")


@dataclass(frozen=True)
class Gemma3Config:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    query_pre_attn_scalar: float
    rms_norm_eps: float
    rope_theta: float
    rope_local_base_freq: float
    rope_scaling_factor: float
    sliding_window: Optional[int]
    layer_is_sliding: Tuple[bool, ...]
    tie_word_embeddings: bool
    max_position_embeddings: int
    bos_token_id: Optional[int]
    eos_token_ids: Tuple[int, ...]

    architecture = "Gemma3ForCausalLM"

    # ------------------------------------------------------------------ parse
    @classmethod
    def from_dict(cls, raw: dict) -> "Gemma3Config":
        c = dict(raw)
        if isinstance(raw.get("text_config"), dict):
            c.update(raw["text_config"])

        def need_int(key: str) -> int:
            if c.get(key) is None:
                raise ConfigError(f"config.json: required key '{key}' is missing")
            v = c[key]
            if isinstance(v, bool) or not isinstance(v, (int, float)) or int(v) != v or int(v) < 1:
                raise ConfigError(f"config.json: '{key}' must be a positive integer, got {v!r}")
            return int(v)

        def opt_float(key: str) -> float:
            v = c.get(key)
            if v is None:
                v = _OPTIONAL_DEFAULTS[key]
            if isinstance(v, bool) or not isinstance(v, (int, float)) or not math.isfinite(v) or v <= 0:
                raise ConfigError(f"config.json: '{key}' must be a positive number, got {v!r}")
            return float(v)

        vocab = need_int("vocab_size")
        hidden = need_int("hidden_size")
        n_layers = need_int("num_hidden_layers")
        n_heads = need_int("num_attention_heads")
        n_kv = need_int("num_key_value_heads")
        head_dim = need_int("head_dim")
        inter = need_int("intermediate_size")
        if n_heads % n_kv != 0:
            raise ConfigError(f"config.json: num_attention_heads ({n_heads}) is not a multiple of "
                              f"num_key_value_heads ({n_kv})")
        if head_dim % 2 != 0:
            raise ConfigError(f"config.json: head_dim ({head_dim}) must be even for the rotation of pairs")

        act = c.get("hidden_activation", c.get("hidden_act"))
        if act is not None and act not in ("gelu_pytorch_tanh", "gelu_tanh"):
            raise ConfigError(f"config.json: unsupported hidden_activation {act!r} (only gelu_pytorch_tanh)")
        for key in ("final_logit_softcapping", "attn_logit_softcapping"):
            if c.get(key) not in (None, 0, 0.0):
                raise ConfigError(f"config.json: unsupported {key}={c[key]!r} (the reference fixes it off, "
                                  f"src/models/gemma3.zig:197)")
        if c.get("attention_bias"):
            raise ConfigError("config.json: unsupported attention_bias=true (no tensor has a bias)")

        scalar = c.get("query_pre_attn_scalar")
        if scalar is None:
            scalar = head_dim                               # gemma3.zig:190-194
        if isinstance(scalar, bool) or not isinstance(scalar, (int, float)) or scalar <= 0:
            raise ConfigError(f"config.json: query_pre_attn_scalar must be positive, got {scalar!r}")

        # per-layer kind: layer_types wins, else every pattern-th layer is global (gemma3.zig:736)
        if c.get("layer_types") is not None:
            lt = c["layer_types"]
            if not isinstance(lt, list) or len(lt) != n_layers:
                raise ConfigError(f"config.json: layer_types must list {n_layers} entries")
            bad = [t for t in lt if t not in ("sliding_attention", "full_attention")]
            if bad:
                raise ConfigError(f"config.json: unknown layer type {bad[0]!r}")
            sliding = tuple(t == "sliding_attention" for t in lt)
        else:
            pattern = c.get("sliding_window_pattern")
            if pattern is None:
                pattern = _OPTIONAL_DEFAULTS["sliding_window_pattern"]
            if isinstance(pattern, bool) or not isinstance(pattern, int) or pattern < 0:
                raise ConfigError(f"config.json: sliding_window_pattern must be an integer >= 0, got {pattern!r}")
            sliding = tuple(pattern > 0 and (i + 1) % pattern != 0 for i in range(n_layers))

        window = c.get("sliding_window")
        if any(sliding):
            if window is None:
                raise ConfigError("config.json: required key 'sliding_window' is missing "
                                  "(some layers are sliding_attention)")
            if isinstance(window, bool) or not isinstance(window, int) or window < 1:
                raise ConfigError(f"config.json: sliding_window must be an integer >= 1, got {window!r}")
        else:
            window = None

        factor = 1.0
        theta_g, theta_l = opt_float("rope_theta"), opt_float("rope_local_base_freq")
        scaling = c.get("rope_scaling")
        params = c.get("rope_parameters")
        if isinstance(params, dict) and ("full_attention" in params or "sliding_attention" in params):
            full = params.get("full_attention") or {}
            local = params.get("sliding_attention") or {}
            theta_g = float(full.get("rope_theta", theta_g))
            theta_l = float(local.get("rope_theta", theta_l))
            scaling = full
            if (local.get("rope_type") or "default") != "default":
                raise ConfigError("config.json: rope scaling on sliding layers is unsupported")
        if scaling:
            kind = scaling.get("rope_type", scaling.get("type", "default"))
            if kind == "linear":
                factor = float(scaling.get("factor", 1.0))
                if not math.isfinite(factor) or factor <= 0:
                    raise ConfigError(f"config.json: rope_scaling.factor must be positive, got {factor!r}")
            elif kind != "default":
                raise ConfigError(f"config.json: unsupported rope_scaling type {kind!r} (only linear)")

        eos = c.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, list):
            eos_ids = tuple(int(x) for x in eos)
        else:
            eos_ids = (int(eos),)
        bos = c.get("bos_token_id")

        max_pos = c.get("max_position_embeddings")
        if max_pos is None:
            max_pos = _OPTIONAL_DEFAULTS["max_position_embeddings"]

        return cls(
            vocab_size=vocab, hidden_size=hidden, num_hidden_layers=n_layers,
            num_attention_heads=n_heads, num_key_value_heads=n_kv, head_dim=head_dim,
            intermediate_size=inter, query_pre_attn_scalar=float(scalar),
            rms_norm_eps=opt_float("rms_norm_eps"), rope_theta=theta_g,
            rope_local_base_freq=theta_l, rope_scaling_factor=factor,
            sliding_window=window, layer_is_sliding=sliding,
            tie_word_embeddings=bool(c.get("tie_word_embeddings", True)),
            max_position_embeddings=int(max_pos),
            bos_token_id=None if bos is None else int(bos), eos_token_ids=eos_ids)

    # ------------------------------------------------------------------ export
    def to_dict(self) -> dict:
        """config.json content that parses back to this configuration."""
        d = {
            "architectures": [self.architecture], "model_type": "gemma3_text",
            "vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads, "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "query_pre_attn_scalar": self.query_pre_attn_scalar,
            "rms_norm_eps": self.rms_norm_eps, "rope_theta": self.rope_theta,
            "rope_local_base_freq": self.rope_local_base_freq,
            "rope_scaling": ({"rope_type": "linear", "factor": self.rope_scaling_factor}
                             if self.rope_scaling_factor != 1.0 else None),
            "sliding_window": self.sliding_window,
            "layer_types": ["sliding_attention" if s else "full_attention" for s in self.layer_is_sliding],
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_activation": "gelu_pytorch_tanh",
            "max_position_embeddings": self.max_position_embeddings,
            "bos_token_id": self.bos_token_id,
            "eos_token_id": list(self.eos_token_ids) if len(self.eos_token_ids) != 1 else self.eos_token_ids[0],
        }
        return d

    # ------------------------------------------------------------------ spec
    def model_spec(self, tensor_names: Optional[Iterable[str]] = None) -> ModelSpec:
        """The architecture as parts.  ``tensor_names`` (the names a checkpoint holds)
        pick the name prefix (src/format/safetensors.zig:517-521) and whether a separate
        output matrix exists (src/models/gemma3.zig:357-358)."""
        names = set(tensor_names) if tensor_names is not None else None
        p = "model."
        if names is not None:
            for cand in TENSOR_PREFIXES:
                if cand + "embed_tokens.weight" in names:
                    p = cand
                    break
        if names is not None and "lm_head.weight" in names:
            head: Optional[str] = "lm_head.weight"
        elif self.tie_word_embeddings:
            head = None
        else:
            head = "lm_head.weight"          # untied and absent: the loader reports it missing

        e, hd, eps = self.hidden_size, self.head_dim, self.rms_norm_eps

        def norm(name: str, size: int) -> NormSpec:
            return NormSpec("rmsnorm", size, eps, name, add_one=True)    # gemma3.zig:943-949

        layers: List[LayerSpec] = []
        for i, sliding in enumerate(self.layer_is_sliding):
            lp = f"{p}layers.{i}."
            pos = PositionSpec(
                "rope", rotary_dim=hd,                                    # gemma3.zig:157
                theta=self.rope_local_base_freq if sliding else self.rope_theta,
                factor=1.0 if sliding else self.rope_scaling_factor)      # gemma3.zig:736-748
            mixer = AttentionSpec(
                kind="attention", hidden=e, n_heads=self.num_attention_heads,
                n_kv_heads=self.num_key_value_heads, head_dim=hd,
                scale=1.0 / math.sqrt(self.query_pre_attn_scalar),        # gemma3.zig:190-194
                window=self.sliding_window if sliding else None, position=pos,
                q_norm=norm(lp + "self_attn.q_norm.weight", hd),
                k_norm=norm(lp + "self_attn.k_norm.weight", hd),
                q_proj=lp + "self_attn.q_proj.weight", k_proj=lp + "self_attn.k_proj.weight",
                v_proj=lp + "self_attn.v_proj.weight", o_proj=lp + "self_attn.o_proj.weight")
            ffn = GatedFfnSpec(
                kind="gated_dense", hidden=e, intermediate=self.intermediate_size,
                activation="gelu_tanh", gate_proj=lp + "mlp.gate_proj.weight",
                up_proj=lp + "mlp.up_proj.weight", down_proj=lp + "mlp.down_proj.weight")
            layers.append(LayerSpec(
                kind="sandwich", mixer=mixer, ffn=ffn,
                pre_mixer_norm=norm(lp + "input_layernorm.weight", e),
                post_mixer_norm=norm(lp + "post_attention_layernorm.weight", e),
                pre_ffn_norm=norm(lp + "pre_feedforward_layernorm.weight", e),
                post_ffn_norm=norm(lp + "post_feedforward_layernorm.weight", e)))
        return ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab_size, hidden=e,
            embed_weight=p + "embed_tokens.weight",
            embed_scale=math.sqrt(float(e)),                              # gemma3.zig:195
            layers=layers, order=[RunEntry(i, i, True) for i in range(len(layers))],
            final_norm=norm(p + "norm.weight", e), head_weight=head,
            max_context=self.max_position_embeddings, bos_token_id=self.bos_token_id,
            eos_token_ids=self.eos_token_ids,
            # what the reference's lookup can reach: names under the chosen prefix and the
            # top-level output matrix (safetensors.zig:333-349, 535-540)
            tensor_scope=(p, "lm_head."))
