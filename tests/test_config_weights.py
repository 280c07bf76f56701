"""Configuration, registries and weight loading errors (no GPU)."""
import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

import tiny
from simply_amd import registry
from simply_amd.config import ConfigError, Gemma2Config, config_from_dict, load_config
from simply_amd.models import DecoderModel
from simply_amd.weights import WeightsError, load_weights, write_random_model
from simply_amd.weights.loader import target_dtype
from simply_amd.parts.base import ParamSpec


def test_reads_every_key():
    c = config_from_dict(tiny.TINY_B)
    assert isinstance(c, Gemma2Config)
    assert (c.hidden_size, c.num_hidden_layers, c.num_attention_heads, c.num_key_value_heads, c.head_dim,
            c.intermediate_size, c.vocab_size) == (96, 3, 6, 1, 32, 320, 512)
    assert c.rms_norm_eps == 1e-5 and c.rope_theta == 1e6 and c.query_pre_attn_scalar == 24
    assert c.sliding_window == 16 and c.attn_logit_softcapping is None and c.final_logit_softcapping == 15.0
    assert c.layer_types == ("sliding_attention", "full_attention", "sliding_attention")
    spec = c.model_spec()
    assert [l.mixer.params["window"] for l in spec.layers] == [16, None, 16]
    assert spec.layers[0].mixer.params["query_scale"] == pytest.approx(24 ** 0.5)
    assert spec.layers[0].mixer.params["soft_cap"] is None and spec.head.params["soft_cap"] == 15.0
    assert spec.embedding.params["scale"] == pytest.approx(96 ** 0.5)
    assert spec.head.tensors["weight"] == "model.embed_tokens.weight"
    # round trip through config.json
    assert config_from_dict(c.to_dict()) == c


def test_defaults_are_gemma2s():
    d = {k: v for k, v in tiny.TINY_A.items() if k in ("architectures", "hidden_size", "num_hidden_layers",
         "num_attention_heads", "num_key_value_heads", "head_dim", "intermediate_size", "vocab_size")}
    c = config_from_dict(d)
    assert (c.rms_norm_eps, c.rope_theta, c.sliding_window, c.attn_logit_softcapping, c.final_logit_softcapping,
            c.query_pre_attn_scalar, c.tie_word_embeddings) == (1e-6, 10000.0, 4096, 50.0, 30.0, 16.0, True)
    assert c.layer_types == ("sliding_attention", "full_attention")   # even layers are windowed


@pytest.mark.parametrize("change,match", [
    ({"architectures": ["NoSuchModel"]}, "unknown architecture"),
    ({"architectures": []}, "architectures"),
    ({"hidden_size": None}, "hidden_size"),
    ({"num_attention_heads": 5}, "multiple"),
    ({"head_dim": 15}, "even"),
    ({"hidden_activation": "relu"}, "hidden_activation"),
    ({"layer_types": ["full_attention"]}, "layer_types"),
    ({"layer_types": ["full_attention", "banana"]}, "unknown layer type"),
    ({"attention_bias": True}, "attention_bias"),
    ({"vocab_size": 0}, "positive"),
])
def test_bad_configs_are_refused(change, match):
    d = dict(tiny.TINY_A)
    d.update(change)
    with pytest.raises(ValueError, match=match):
        config_from_dict(d)


def test_untied_head_and_no_window():
    d = dict(tiny.TINY_A, tie_word_embeddings=False, sliding_window=None)
    spec = config_from_dict(d).model_spec()
    assert spec.head.tensors["weight"] == "lm_head.weight"
    assert all(l.mixer.params["window"] is None for l in spec.layers)
    assert "lm_head.weight" in DecoderModel(spec).expected_tensors()


def test_registry_rules():
    r = registry.Registry("thing")
    r.register("a", 1)
    with pytest.raises(ValueError, match="duplicate"):
        r.register("a", 2)
    with pytest.raises(ValueError, match="known: a"):
        r.get("b")
    assert "Gemma2ForCausalLM" in registry.ARCHITECTURES and "paged_attention" in registry.MIXERS


def test_schedule_validation():
    import dataclasses
    from simply_amd.config import ScheduleEntry
    spec = config_from_dict(tiny.TINY_A).model_spec()
    for bad in ([ScheduleEntry(5)], [ScheduleEntry(0, cache_from=0)], [ScheduleEntry(0), ScheduleEntry(1, 0), ScheduleEntry(0, 1)]):
        with pytest.raises(ValueError):
            dataclasses.replace(spec, schedule=tuple(bad)).validate()
    dataclasses.replace(spec, schedule=(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0, 0), ScheduleEntry(1))).validate()


def test_random_folder_round_trip(tmp_path):
    d = tiny.write_model("A", str(tmp_path / "A"), dtype=torch.bfloat16)
    assert sorted(os.listdir(d)) == ["config.json", "model.safetensors"]
    cfg = load_config(d)
    model = DecoderModel(cfg.model_spec())
    load_weights(model, d, torch.bfloat16, "cpu")
    stored = load_file(os.path.join(d, "model.safetensors"))
    assert set(stored) == set(model.expected_tensors())
    assert all(t.dtype == torch.bfloat16 for t in stored.values())
    q, k, v = (stored[f"model.layers.1.self_attn.{n}_proj.weight"] for n in "qkv")
    assert torch.equal(model.layers[1].mixer.qkv_proj, torch.cat([q, k, v]))
    assert model.embedding.table is not None and model.head.weight is model.embedding.table  # tied
    # same seed, same weights; the norm scales are not zero
    d2 = tiny.write_model("A", str(tmp_path / "A2"), dtype=torch.bfloat16)
    assert all(torch.equal(a, load_file(os.path.join(d2, "model.safetensors"))[n]) for n, a in stored.items())
    assert stored["model.norm.weight"].float().abs().mean() > 0.01


def test_weight_errors_list_everything(tmp_path):
    d = tiny.write_model("A", str(tmp_path / "A"))
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    del t["model.layers.0.mlp.up_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.7.extra.weight"] = torch.zeros(3)
    t["model.layers.1.self_attn.o_proj.weight"] = torch.zeros(5, 7)
    save_file(t, path)
    model = DecoderModel(load_config(d).model_spec())
    with pytest.raises(WeightsError) as e:
        load_weights(model, d, torch.float32, "cpu")
    msg = str(e.value)
    assert e.value.missing == ["model.layers.0.mlp.up_proj.weight", "model.norm.weight"]
    assert e.value.unexpected == ["model.layers.7.extra.weight"]
    assert e.value.wrong_shape == [("model.layers.1.self_attn.o_proj.weight", (5, 7), (64, 64))]
    for name in ("up_proj", "model.norm.weight", "model.layers.7.extra.weight", "[5, 7]", "[64, 64]"):
        assert name in msg


def test_missing_files(tmp_path):
    with pytest.raises(FileNotFoundError, match="config.json"):
        load_config(str(tmp_path))
    d = tiny.write_model("A", str(tmp_path / "A"))
    os.remove(os.path.join(d, "model.safetensors"))
    with pytest.raises(FileNotFoundError, match="model.safetensors"):
        load_weights(DecoderModel(load_config(d).model_spec()), d, torch.float32, "cpu")


def test_sharded_files_and_duplicates(tmp_path):
    d = tiny.write_model("A", str(tmp_path / "A"))
    t = load_file(os.path.join(d, "model.safetensors"))
    os.remove(os.path.join(d, "model.safetensors"))
    names = sorted(t)
    save_file({n: t[n] for n in names[:5]}, os.path.join(d, "model-00001-of-00002.safetensors"))
    save_file({n: t[n] for n in names[5:]}, os.path.join(d, "model-00002-of-00002.safetensors"))
    model = DecoderModel(load_config(d).model_spec())
    load_weights(model, d, torch.float32, "cpu")
    assert torch.equal(model.final_norm.scale, t["model.norm.weight"])
    save_file({n: t[n] for n in names[4:]}, os.path.join(d, "model-00002-of-00002.safetensors"))
    with pytest.raises(WeightsError, match="more than one file"):
        load_weights(model, d, torch.float32, "cpu")


def test_element_types():
    m, v, tb = ParamSpec((2, 2)), ParamSpec((2,), role="vector"), ParamSpec((2,), role="table")
    bf, f32 = torch.bfloat16, torch.float32
    assert target_dtype(bf, m, bf) == bf and target_dtype(f32, m, bf) == bf      # matrices in the activation dtype
    assert target_dtype(f32, v, bf) == f32 and target_dtype(bf, v, bf) == bf      # a 32-bit stored vector stays so
    assert target_dtype(bf, m, f32) == f32 and target_dtype(bf, v, f32) == f32    # the 32-bit path holds 32-bit
    assert target_dtype(torch.int64, tb, bf) == torch.int32 and target_dtype(torch.int32, m, f32) == torch.int32
