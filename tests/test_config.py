"""Configuration: the typed Qwen3 configuration read from config.json keys, and the registry."""
import json

import pytest
import torch

import configs
from lucciola_amd import models  # noqa: F401  (registers the architectures)
from lucciola_amd.config.engine_config import EngineConfig, parse_dtype
from lucciola_amd.config.model_config import ConfigError, Qwen3Config, read_config_json
from lucciola_amd.config.registry import (ARCHITECTURES, MIXERS, Architecture, RegistryError,
                                          architecture_for)
from lucciola_amd.config.specs import RunEntry


def test_reads_every_key():
    cfg = Qwen3Config.from_dict(configs.TINY_B)
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads) == (3, 96, 8)
    assert (cfg.num_key_value_heads, cfg.head_dim, cfg.intermediate_size, cfg.vocab_size) == (1, 32, 160, 384)
    assert cfg.rope_theta == 1e6 and cfg.rms_norm_eps == 1e-5 and cfg.tie_word_embeddings is False
    assert cfg.initializer_range == 0.05 and cfg.max_position_embeddings == 2048
    assert cfg.sliding_window is None and set(cfg.layer_types) == {"full_attention"}


def test_defaults_follow_the_reference():
    # src/qwen.cc:53-56: kv heads default to the heads, head_dim to hidden / heads
    cfg = Qwen3Config.from_dict({"architectures": ["Qwen3ForCausalLM"], "hidden_size": 64,
                                 "num_attention_heads": 4, "num_hidden_layers": 2,
                                 "intermediate_size": 128, "vocab_size": 100})
    assert cfg.num_key_value_heads == 4 and cfg.head_dim == 16
    assert cfg.rms_norm_eps == 1e-6 and cfg.rope_theta == 1e6 and not cfg.tie_word_embeddings


@pytest.mark.parametrize("key", ["hidden_size", "num_attention_heads", "num_hidden_layers",
                                 "intermediate_size", "vocab_size"])
def test_missing_key_is_an_error(key):
    data = dict(configs.TINY_A)
    del data[key]
    with pytest.raises(ConfigError, match=key):
        Qwen3Config.from_dict(data)


@pytest.mark.parametrize("change,needle", [
    ({"num_key_value_heads": 3}, "multiple"), ({"head_dim": 15}, "even"),
    ({"rms_norm_eps": 0.0}, "rms_norm_eps"), ({"hidden_act": "gelu"}, "hidden_act"),
    ({"attention_bias": True}, "attention_bias"), ({"vocab_size": 0}, "vocab_size"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 4.0}}, "rope_scaling"),
    ({"layer_types": ["full_attention"]}, "layer_types"),
    ({"layer_types": ["full_attention", "sliding_attention"]}, "sliding_window"),
    ({"hidden_size": "64"}, "integer")])
def test_bad_values_are_refused(change, needle):
    with pytest.raises(ConfigError, match=needle):
        Qwen3Config.from_dict(dict(configs.TINY_A, **change))


def test_sliding_window_layers():
    cfg = Qwen3Config.from_dict(configs.TINY_C)
    assert cfg.sliding_window == 24
    assert cfg.layer_types == ("full_attention", "sliding_attention", "full_attention", "sliding_attention")
    # the older spelling: layers from max_window_layers on slide
    data = {k: v for k, v in configs.TINY_C.items() if k != "layer_types"}
    data["max_window_layers"] = 3
    assert Qwen3Config.from_dict(data).layer_types == ("full_attention",) * 3 + ("sliding_attention",)
    data["use_sliding_window"] = False
    off = Qwen3Config.from_dict(data)
    assert off.sliding_window is None and set(off.layer_types) == {"full_attention"}


@pytest.mark.parametrize("key", ["A", "B", "C", "D"])
def test_round_trip(key, tmp_path):
    cfg = Qwen3Config.from_dict(configs.ALL[key][0])
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
    assert Qwen3Config.from_folder(str(tmp_path)) == cfg


def test_folder_errors(tmp_path):
    with pytest.raises(ConfigError, match="no config.json"):
        read_config_json(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        read_config_json(str(tmp_path))


def test_registry_names_the_model_and_lists_known_names():
    arch = architecture_for(configs.TINY_A)
    assert arch.name == "Qwen3ForCausalLM"
    with pytest.raises(RegistryError, match="Qwen3ForCausalLM"):
        architecture_for({"architectures": ["NoSuchModel"]})
    with pytest.raises(RegistryError, match="architectures"):
        architecture_for({})
    with pytest.raises(RegistryError, match="attention"):
        MIXERS.get("nothing")


def test_registering_another_architecture():
    arch = Architecture("ToyForCausalLM", read_config=lambda d: d, model_spec=lambda c: None)
    ARCHITECTURES.register("ToyForCausalLM", arch)
    try:
        assert architecture_for({"architectures": ["ToyForCausalLM"]}) is arch
        with pytest.raises(RegistryError, match="already registered"):
            ARCHITECTURES.register("ToyForCausalLM", Architecture("x", None, None))
    finally:
        ARCHITECTURES.unregister("ToyForCausalLM")


def test_model_spec_is_data():
    arch = architecture_for(configs.TINY_C)
    spec = arch.model_spec(arch.read_config(configs.TINY_C))
    assert [e.layer for e in spec.run_order] == [0, 1, 2, 3]
    assert [l.parts["mixer"].params["window"] for l in spec.layers] == [None, 24, None, 24]
    assert spec.layers[0].parts["mixer"].params["qk_norm"].params == {"size": 48, "eps": 3e-6}
    assert spec.layers[2].names["mixer.q_proj"] == "model.layers.2.self_attn.q_proj.weight"
    assert spec.head_name == "lm_head.weight"
    assert sorted(spec.layers[0].parts) == ["feed_forward", "feed_forward_norm", "mixer", "mixer_norm"]
    tied = arch.model_spec(arch.read_config(configs.TINY_A))
    assert tied.head_name is None
    # the run order is checked
    from dataclasses import replace
    with pytest.raises(ValueError, match="earlier site"):
        replace(spec, run_order=[RunEntry(0, cache_of=0)]).validate()
    with pytest.raises(ValueError, match="names layer"):
        replace(spec, run_order=[RunEntry(9)]).validate()


def test_engine_config():
    assert parse_dtype("bf16") is torch.bfloat16 and parse_dtype("float32") is torch.float32
    with pytest.raises(ValueError):
        parse_dtype("float16")
    with pytest.raises(ValueError):
        EngineConfig(block_size=0)
    assert EngineConfig(dtype="fp32").dtype is torch.float32
