"""Configuration and registry: config.json's own keys, errors that name the key."""
import json
import math

import pytest

import plain_gemma3 as P
from agave_amd.config import (ConfigError, Gemma3Config, UnsupportedArchitecture, architectures,
                              find_architecture, load_config)


def test_tiny_configs_parse_and_differ():
    a = Gemma3Config.from_dict(P.tiny_config("A"))
    b = Gemma3Config.from_dict(P.tiny_config("B"))
    assert a.layer_is_sliding == (True, False, True, False)
    assert b.layer_is_sliding == (True, True, False, True, True, False)
    assert (a.query_pre_attn_scalar, b.query_pre_attn_scalar) == (32.0, 16.0)
    assert (a.rope_scaling_factor, b.rope_scaling_factor) == (1.0, 8.0)
    assert b.eos_token_ids == (1, 106) and a.eos_token_ids == (1,)
    for f in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads",
              "head_dim", "intermediate_size", "rms_norm_eps", "rope_theta", "rope_local_base_freq", "sliding_window"):
        assert getattr(a, f) != getattr(b, f), f


def test_spec_carries_every_constant():
    cfg = Gemma3Config.from_dict(P.tiny_config("B"))
    spec = cfg.model_spec()
    assert spec.embed_scale == pytest.approx(math.sqrt(96))
    sliding, full = spec.layers[0].mixer, spec.layers[2].mixer
    assert sliding.window == 8 and full.window is None
    assert sliding.position.theta == 1e3 and sliding.position.factor == 1.0
    assert full.position.theta == 5e5 and full.position.factor == 8.0
    assert full.scale == pytest.approx(1 / math.sqrt(16))
    assert spec.layers[0].pre_mixer_norm.eps == 1e-5 and spec.layers[0].pre_mixer_norm.add_one
    assert [e.layer for e in spec.order] == list(range(6))
    assert spec.head_weight is None


def test_text_config_overrides_and_layer_types():
    raw = {"architectures": ["Gemma3ForConditionalGeneration"], "model_type": "gemma3", "hidden_size": 1,
           "text_config": dict(P.tiny_config("C"), model_type="gemma3_text")}
    arch = find_architecture(raw)
    cfg = arch.parse(raw)
    assert cfg.hidden_size == 160
    assert cfg.layer_is_sliding == (True, False, True, True, False)
    assert not cfg.tie_word_embeddings
    spec = arch.spec(cfg, ["model.language_model.embed_tokens.weight", "lm_head.weight"])
    assert spec.embed_weight == "model.language_model.embed_tokens.weight"
    assert spec.head_weight == "lm_head.weight"


def test_round_trip_through_to_dict():
    for which in "ABC":
        cfg = Gemma3Config.from_dict(P.tiny_config(which))
        assert Gemma3Config.from_dict(cfg.to_dict()) == cfg


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                                 "num_key_value_heads", "head_dim", "intermediate_size", "sliding_window"])
def test_missing_size_names_the_key(key):
    raw = P.tiny_config("A")
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        Gemma3Config.from_dict(raw)


@pytest.mark.parametrize("patch,word", [
    ({"num_key_value_heads": 3}, "multiple"), ({"head_dim": 33}, "even"),
    ({"hidden_activation": "silu"}, "hidden_activation"), ({"final_logit_softcapping": 30.0}, "final_logit_softcapping"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "yarn"), ({"sliding_window": 0}, "sliding_window"),
    ({"layer_types": ["full_attention"]}, "layer_types"), ({"vocab_size": -5}, "vocab_size"),
    ({"rms_norm_eps": 0}, "rms_norm_eps")])
def test_bad_values(patch, word):
    with pytest.raises(ConfigError, match=word):
        Gemma3Config.from_dict(dict(P.tiny_config("A"), **patch))


def test_optional_keys_fall_back_as_the_reference():
    raw = P.tiny_config("A")
    for k in ("query_pre_attn_scalar", "rope_theta", "rope_local_base_freq", "rms_norm_eps", "sliding_window_pattern"):
        raw.pop(k)
    cfg = Gemma3Config.from_dict(raw)
    assert cfg.query_pre_attn_scalar == cfg.head_dim           # src/models/gemma3.zig:190-194
    assert (cfg.rope_theta, cfg.rope_local_base_freq, cfg.rms_norm_eps) == (1e6, 1e4, 1e-6)
    assert cfg.layer_is_sliding == (True, True, True, True)    # pattern 6 on four layers: none is global


def test_registry(tmp_path):
    assert "Gemma3ForCausalLM" in architectures()
    assert find_architecture({"model_type": "gemma3_text"}).name == "Gemma3ForCausalLM"
    with pytest.raises(UnsupportedArchitecture, match="LlamaForCausalLM.*supported.*Gemma3ForCausalLM"):
        find_architecture({"architectures": ["LlamaForCausalLM"], "model_type": "llama"})
    with pytest.raises(ConfigError, match="not found"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="JSON"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps(P.tiny_config("A")))
    arch, cfg = load_config(str(tmp_path))
    assert arch.name == "Gemma3ForCausalLM" and cfg.vocab_size == 512
