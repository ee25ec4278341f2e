"""Configuration: typed reading of config.json keys, defaults, refusals, and the registry."""
import copy

import pytest

from axon_amd.config import (ConfigError, Qwen2Config, architecture_of, config_from_dict, known_architectures,
                             register_architecture)
from helpers import TINY


def test_reads_every_size_from_config_json():
    for name in TINY:
        c = TINY[name]["config"]
        cfg = config_from_dict(c)
        assert isinstance(cfg, Qwen2Config)
        assert cfg.num_hidden_layers == c["num_hidden_layers"] and cfg.hidden_size == c["hidden_size"]
        assert cfg.intermediate_size == c["intermediate_size"] and cfg.vocab_size == c["vocab_size"]
        assert cfg.num_attention_heads == c["num_attention_heads"]
        assert cfg.num_key_value_heads == c["num_key_value_heads"]
        assert cfg.head_dim == c.get("head_dim", c["hidden_size"] // c["num_attention_heads"])
        assert cfg.rope_theta == c["rope_theta"] and cfg.rms_norm_eps == c["rms_norm_eps"]
        assert cfg.tie_word_embeddings == c["tie_word_embeddings"]
        assert config_from_dict(cfg.to_dict()) == cfg                      # round trip through its own keys


def test_defaults_are_the_references():
    c = {k: v for k, v in TINY["A"]["config"].items() if k not in ("rope_theta", "rms_norm_eps", "tie_word_embeddings")}
    cfg = config_from_dict(c)
    assert cfg.rope_theta == 10000.0 and cfg.rms_norm_eps == 1e-6 and cfg.tie_word_embeddings is False
    c["rope_parameters"] = {"rope_theta": 5e5, "rope_type": "default"}
    assert config_from_dict(c).rope_theta == 5e5


def test_model_spec_carries_the_constants():
    cfg = config_from_dict(TINY["B"]["config"])
    spec = cfg.model_spec()
    assert len(spec.layers) == 3 and [r.layer for r in spec.order] == [0, 1, 2]
    mixer = spec.layers[1].mixer
    assert mixer.kind == "gqa_attention" and mixer.params["num_kv_heads"] == 1 and mixer.params["head_dim"] == 32
    assert mixer.params["position"].params["theta"] == 1000000.0
    assert spec.layers[0].norm.params["eps"] == 1e-5 and spec.head.params["tied"] is False
    assert spec.layers[2].prefix == "model.layers.2."


@pytest.mark.parametrize("edit,fragment", [
    ({"hidden_act": "gelu"}, "hidden_act gelu is not supported"),
    ({"use_sliding_window": True}, "use_sliding_window true is not supported"),
    ({"quantization_config": {"quant_method": "fp8"}}, "quantization_config"),
    ({"rope_scaling": {"type": "yarn", "factor": 4.0}}, "RoPE scaling type yarn is not supported"),
    ({"num_key_value_heads": None}, "missing num_key_value_heads"),
    ({"num_hidden_layers": 2.5}, "is not a whole number"),
    ({"num_hidden_layers": 0}, "at least 1"),
    ({"num_attention_heads": 3}, "not a multiple of num_attention_heads"),
    ({"num_key_value_heads": 3}, "not a multiple of num_key_value_heads"),
    ({"head_dim": 15}, "odd"),
    ({"rms_norm_eps": -1.0}, "must be above 0"),
    ({"tie_word_embeddings": "yes"}, "is not true or false"),
    ({"model_type": "mamba", "architectures": ["MambaForCausalLM"]}, "is not supported"),
])
def test_refusals(edit, fragment):
    c = copy.deepcopy(TINY["A"]["config"])
    for k, v in edit.items():
        if v is None:
            c.pop(k, None)
        else:
            c[k] = v
    with pytest.raises(ConfigError) as e:
        config_from_dict(c)
    assert fragment in str(e.value)


def test_registry_finds_by_architecture_or_model_type():
    assert "Qwen2ForCausalLM" in known_architectures()
    assert architecture_of({"model_type": "qwen2"}) == "Qwen2ForCausalLM"
    assert architecture_of({"architectures": ["Qwen2ForCausalLM"]}) == "Qwen2ForCausalLM"

    class Other(Qwen2Config):
        architecture = "OtherForCausalLM"

    register_architecture("OtherForCausalLM", Other, "other")
    c = dict(TINY["A"]["config"], architectures=["OtherForCausalLM"], model_type="other")
    assert type(config_from_dict(c)) is Other


def test_engine_config():
    from axon_amd.config import EngineConfig
    assert EngineConfig(dtype="bf16").dtype == "bfloat16" and EngineConfig(dtype="fp32").dtype == "float32"
    with pytest.raises(ConfigError):
        EngineConfig(dtype="float16")
    with pytest.raises(ConfigError):
        EngineConfig(page_size=0)


def test_theta_is_kept_as_a_32_bit_float_and_a_quantized_export_is_refused(tmp_path):
    import json
    import struct
    from axon_amd.config import ConfigError, config_from_dict, read_config_json
    base = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=1, hidden_size=64, intermediate_size=64,
                num_attention_heads=2, num_key_value_heads=1, vocab_size=32, max_position_embeddings=64)
    # src/safetensors.rs:649-651: a base that 32 bits cannot hold is rounded to the nearest that they can
    theta = 1000003.7
    c = config_from_dict(dict(base, rope_theta=theta))
    assert c.rope_theta == struct.unpack("<f", struct.pack("<f", theta))[0] != theta
    assert config_from_dict(dict(base, rope_theta=1000000.0)).rope_theta == 1000000.0
    # src/safetensors.rs:1444-1449
    (tmp_path / "config.json").write_text(json.dumps(base))
    assert read_config_json(str(tmp_path))["hidden_size"] == 64
    (tmp_path / "hf_quant_config.json").write_text("{}")
    with pytest.raises(ConfigError, match="hf_quant_config.json"):
        read_config_json(str(tmp_path))
