"""Weights: the container's reader against another writer, the round trip of the random-weights
mode, and the one error that lists everything wrong."""
import json
import os
import struct

import pytest
import torch

import plain_gemma3 as P
from agave_amd.config import find_architecture
from agave_amd.engine.model import tensor_needs
from agave_amd.weights import (Checkpoint, DictWeightSource, SafetensorsError, TensorNeed, WeightError,
                               WeightSource, check_tensors, write_random_model, write_safetensors)


def _needs(which="A"):
    raw = P.tiny_config(which)
    arch = find_architecture(raw)
    return raw, tensor_needs(arch.spec(arch.parse(raw), None))


def test_reader_against_the_safetensors_package(tmp_path):
    from safetensors.torch import save_file
    t = {"a": torch.randn(3, 5).bfloat16(), "b": torch.randn(7), "c": torch.arange(6, dtype=torch.int64).view(2, 3),
         "d": torch.randn(2, 2).half(), "e": torch.zeros(0, 4)}
    save_file(t, str(tmp_path / "model.safetensors"))
    ck = Checkpoint(str(tmp_path))
    assert sorted(ck.names()) == sorted(t)
    assert ck.read("a").dtype == torch.bfloat16 and torch.equal(ck.read("a"), t["a"])
    assert ck.read("b").dtype == torch.float32 and torch.equal(ck.read("b"), t["b"])      # 32-bit stays 32-bit
    assert ck.read("c").dtype == torch.int32 and torch.equal(ck.read("c").long(), t["c"])  # tables as int32
    assert ck.read("d").dtype == torch.float16 and torch.equal(ck.read("d"), t["d"])      # cast where it is used
    assert [ck.stored_dtype(n) for n in "abcd"] == ["BF16", "F32", "I64", "F16"]
    assert ck.read("e").shape == (0, 4)


def test_own_writer_is_read_by_the_package(tmp_path):
    from safetensors.torch import load_file
    t = {"x": torch.randn(4, 3).bfloat16(), "y": torch.randn(5)}
    write_safetensors(str(tmp_path / "m.safetensors"), t)
    back = load_file(str(tmp_path / "m.safetensors"))
    assert torch.equal(back["x"], t["x"]) and torch.equal(back["y"], t["y"])


def test_random_model_round_trip(tmp_path):
    raw, needs = _needs("B")
    write_random_model(raw, 7, str(tmp_path))
    ck = Checkpoint(str(tmp_path))
    src = WeightSource(ck, needs)
    assert json.load(open(tmp_path / "config.json")) == raw
    again = str(tmp_path / "again")
    write_random_model(raw, 7, again)
    other = str(tmp_path / "other")
    write_random_model(raw, 8, other)
    for n in needs:
        a = src.get(n.name)
        assert a.dtype == torch.bfloat16 and tuple(a.shape) == n.shape
        assert torch.equal(a, Checkpoint(again).read(n.name))
    assert not torch.equal(src.get(needs[0].name), Checkpoint(other).read(needs[0].name))
    emb = src.get("model.embed_tokens.weight").float()
    assert 0.015 < float(emb.std()) < 0.025
    assert 0.05 < float(src.get("model.norm.weight").float().std()) < 0.2


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    raw, needs = _needs("A")
    w = P.random_weights(raw, 0)
    del w["model.layers.1.mlp.up_proj.weight"]
    del w["model.norm.weight"]
    w["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(5, 5)
    w["model.layers.9.extra.weight"] = torch.zeros(1)
    with pytest.raises(WeightError) as ei:
        DictWeightSource(w, needs)
    e = ei.value
    assert e.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.9.extra.weight"]
    assert e.wrong_shape == [("model.layers.0.self_attn.q_proj.weight", (5, 5), (128, 64))]
    text = str(e)
    for word in ("missing (2)", "unexpected (1)", "wrong shape (1)", "up_proj", "extra", "[5, 5]", "[128, 64]"):
        assert word in text
    # the same through a folder
    from safetensors.torch import save_file
    save_file({k: v.contiguous() for k, v in w.items()}, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightError, match="missing"):
        WeightSource(Checkpoint(str(tmp_path)), needs)
    check_tensors({"a": (1,)}, [TensorNeed("a", (1,))])


def _wrapped(which, prefix, seed=0):
    """A tiny configuration as the language model of a folder that holds more than it: the
    text keys inside ``text_config``, the decoder's tensors under ``prefix``."""
    inner = P.tiny_config(which)
    raw = {"architectures": ["Gemma3ForConditionalGeneration"], "model_type": "gemma3",
           "text_config": {k: v for k, v in inner.items() if k != "architectures"},
           "vision_config": {"hidden_size": 8}}
    w = {prefix + k[len("model."):] if k.startswith("model.") else k: v
         for k, v in P.random_weights(inner, seed).items()}
    w["vision_tower.vision_model.encoder.layers.0.mlp.fc1.weight"] = torch.zeros(3, 2)
    w["multi_modal_projector.mm_input_projection_weight"] = torch.zeros(2, 2)
    return inner, raw, w


@pytest.mark.parametrize("prefix", ["language_model.model.", "model.language_model."])
def test_a_folder_that_holds_more_than_the_decoder_loads(tmp_path, prefix, capfd):
    """The reference finds a tensor by its name under "model.language_model.", "language_model.model."
    or "model." (src/format/safetensors.zig:333-349, 517-521) and never looks at the others, and
    "gemma3" is one of the model types of this architecture (src/arch.zig:22-23): a vision tower
    and a projector beside the decoder are passed over, and counted; a stray name under the
    decoder's own prefix is still an error."""
    from safetensors.torch import save_file
    inner, raw, w = _wrapped("A", prefix)
    arch = find_architecture(raw)
    cfg = arch.parse(raw)
    assert cfg == arch.parse(inner)
    spec = arch.spec(cfg, w.keys())
    assert spec.embed_weight == prefix + "embed_tokens.weight" and spec.tensor_scope == (prefix, "lm_head.")
    src = DictWeightSource(w, tensor_needs(spec), scope=spec.tensor_scope)
    assert sorted(src.passed_over) == ["multi_modal_projector.mm_input_projection_weight",
                                      "vision_tower.vision_model.encoder.layers.0.mlp.fc1.weight"]
    assert "2 tensors that are not the model's were passed over" in capfd.readouterr().err
    save_file({k: v.bfloat16().contiguous() for k, v in w.items()}, str(tmp_path / "model.safetensors"))
    assert len(WeightSource(Checkpoint(str(tmp_path)), tensor_needs(spec), spec.tensor_scope).passed_over) == 2
    # without a scope every name counts, as for a model that owns its whole folder
    with pytest.raises(WeightError) as ei:
        DictWeightSource(w, tensor_needs(spec))
    assert len(ei.value.unexpected) == 2
    # inside the scope nothing is passed over
    w[prefix + "layers.9.extra.weight"] = torch.zeros(1)
    w["lm_head.bias"] = torch.zeros(1)
    del w[prefix + "norm.weight"]
    with pytest.raises(WeightError) as ei:
        DictWeightSource(w, tensor_needs(spec), scope=spec.tensor_scope)
    assert ei.value.unexpected == sorted(["lm_head.bias", prefix + "layers.9.extra.weight"])
    assert ei.value.missing == [prefix + "norm.weight"]


def test_a_plain_text_folder_owns_every_name_under_its_prefix():
    """With the "model." prefix a foreign tower would sit under another top-level name; anything
    under "model." that no part asked for stays an error."""
    raw, needs = _needs("A")
    arch = find_architecture(raw)
    w = P.random_weights(raw, 0)
    spec = arch.spec(arch.parse(raw), w.keys())
    assert spec.tensor_scope == ("model.", "lm_head.")
    w["model.vision_tower.x"] = torch.zeros(1)
    with pytest.raises(WeightError, match="unexpected"):
        DictWeightSource(w, needs, scope=spec.tensor_scope)
    del w["model.vision_tower.x"]
    w["vision_tower.x"] = torch.zeros(1)
    assert DictWeightSource(w, needs, scope=spec.tensor_scope).passed_over == ["vision_tower.x"]


def test_element_types_are_checked_in_the_same_error(tmp_path):
    """A matrix must be stored as BF16, F16 or F32 (what the reference's loader takes as floats,
    src/format/safetensors.zig:1605-1616); integers, doubles and booleans in its place are listed by
    name in the one error, beside whatever else is wrong."""
    from safetensors.torch import save_file
    raw, needs = _needs("A")
    w = {k: v.bfloat16() for k, v in P.random_weights(raw, 0).items()}
    w["model.layers.0.mlp.up_proj.weight"] = torch.zeros(192, 64, dtype=torch.int32)
    w["model.layers.1.self_attn.q_norm.weight"] = torch.zeros(32, dtype=torch.int64)
    w["model.layers.2.mlp.down_proj.weight"] = torch.zeros(64, 192, dtype=torch.float64)
    w["model.layers.3.self_attn.k_proj.weight"] = w["model.layers.3.self_attn.k_proj.weight"].half()   # fine
    w["model.layers.3.self_attn.v_proj.weight"] = w["model.layers.3.self_attn.v_proj.weight"].float()  # fine
    del w["model.norm.weight"]
    for make in (lambda: DictWeightSource(w, needs),):
        with pytest.raises(WeightError) as ei:
            make()
        e = ei.value
        assert e.missing == ["model.norm.weight"] and not e.unexpected and not e.wrong_shape
        assert sorted(e.wrong_dtype) == [("model.layers.0.mlp.up_proj.weight", "I32", "float"),
                                         ("model.layers.1.self_attn.q_norm.weight", "I64", "float"),
                                         ("model.layers.2.mlp.down_proj.weight", "F64", "float")]
        assert "wrong element type (3)" in str(e) and "stored as I64, needs one of BF16/F16/F32" in str(e)
    save_file({k: v.contiguous() for k, v in w.items()}, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightError) as ei:
        WeightSource(Checkpoint(str(tmp_path)), needs)
    assert len(ei.value.wrong_dtype) == 3 and ei.value.missing == ["model.norm.weight"]
    # an integer table is the other kind of need: floats in its place are refused, wide integers are
    # narrowed only if they fit
    table = TensorNeed("t", (3,), kind="int")
    with pytest.raises(WeightError, match="stored as BF16, needs one of I64/I32/I16/I8/U8"):
        DictWeightSource({"t": torch.zeros(3, dtype=torch.bfloat16)}, [table])
    ok = DictWeightSource({"t": torch.tensor([1, 2, 2 ** 31 - 1])}, [table]).get("t")
    assert ok.dtype == torch.int32 and ok.tolist() == [1, 2, 2 ** 31 - 1]
    with pytest.raises(ValueError, match="do not fit"):
        DictWeightSource({"t": torch.tensor([1, 2, 2 ** 31])}, [table]).get("t")
    save_file({"t": torch.tensor([-5, 2 ** 40, 0])}, str(tmp_path / "wide.safetensors"))
    os.remove(tmp_path / "model.safetensors")
    with pytest.raises(ValueError, match="do not fit"):
        Checkpoint(str(tmp_path)).read("t")


def test_which_element_type_a_matrix_is_held_in():
    """32-bit engines widen everything; a bfloat16 engine keeps bfloat16, casts half precision,
    and keeps 32-bit storage unless told to cast it."""
    from agave_amd.parts import BuildEnv
    f32, bf16, f16 = torch.float32, torch.bfloat16, torch.float16
    env = BuildEnv(bf16, None, None)
    assert [env.weight_dtype(t) for t in (bf16, f16, f32)] == [bf16, bf16, f32]
    env = BuildEnv(bf16, None, None, keep_stored_precision=False)
    assert [env.weight_dtype(t) for t in (bf16, f16, f32)] == [bf16, bf16, bf16]
    env = BuildEnv(f32, None, None)
    assert [env.weight_dtype(t) for t in (bf16, f16, f32)] == [f32, f32, f32]
    with pytest.raises(TypeError):
        env.weight_dtype(torch.int32)


def _raw_file(path, header: bytes, data: bytes = b"", hlen=None):
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(header) if hlen is None else hlen))
        f.write(header)
        f.write(data)


def test_container_errors(tmp_path):
    # mirrors the parser cases of src/format/safetensors.zig:2198-2296
    d = tmp_path
    with pytest.raises(SafetensorsError, match="no .safetensors"):
        Checkpoint(str(d))
    p = str(d / "model.safetensors")
    open(p, "wb").write(b"abc")
    with pytest.raises(SafetensorsError, match="too short"):
        Checkpoint(str(d))
    _raw_file(p, b"{}", hlen=1 << 40)
    with pytest.raises(SafetensorsError, match="exceeds the file"):
        Checkpoint(str(d))
    _raw_file(p, b"{not json")
    with pytest.raises(SafetensorsError, match="JSON"):
        Checkpoint(str(d))
    _raw_file(p, json.dumps({"t": {"dtype": "F32", "shape": [2], "data_offsets": [8, 0]}}).encode(), b"\0" * 8)
    with pytest.raises(SafetensorsError, match="before start"):
        Checkpoint(str(d))
    _raw_file(p, json.dumps({"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}).encode(), b"\0" * 8)
    with pytest.raises(SafetensorsError, match="past the file"):
        Checkpoint(str(d))
    _raw_file(p, json.dumps({"t": {"dtype": "Q4_K", "shape": [2], "data_offsets": [0, 8]}}).encode(), b"\0" * 8)
    with pytest.raises(SafetensorsError, match="unsupported dtype"):
        Checkpoint(str(d))
    _raw_file(p, json.dumps({"t": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}).encode(), b"\0" * 8)
    with pytest.raises(SafetensorsError, match="needs 12 bytes"):
        Checkpoint(str(d))
    _raw_file(p, json.dumps({"__metadata__": {"format": "pt"},
                             "t": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}).encode(),
              struct.pack("<ff", 1.5, -2.0))
    assert Checkpoint(str(d)).read("t").tolist() == [1.5, -2.0]


def test_sharded_folder_with_index(tmp_path):
    from safetensors.torch import save_file
    save_file({"a": torch.ones(2)}, str(tmp_path / "model-00001-of-00002.safetensors"))
    save_file({"b": torch.zeros(3)}, str(tmp_path / "model-00002-of-00002.safetensors"))
    idx = {"weight_map": {"a": "model-00001-of-00002.safetensors", "b": "model-00002-of-00002.safetensors"}}
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(idx))
    ck = Checkpoint(str(tmp_path))
    assert ck.read("a").tolist() == [1, 1] and ck.read("b").tolist() == [0, 0, 0]
    idx["weight_map"]["c"] = "../evil.safetensors"
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(idx))
    with pytest.raises(SafetensorsError, match="bad shard name"):
        Checkpoint(str(tmp_path))
    idx["weight_map"]["c"] = "gone.safetensors"
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(idx))
    with pytest.raises(SafetensorsError, match="not found"):
        Checkpoint(str(tmp_path))
