"""Configuration and registry."""
import json

import pytest

from conftest import TINY
from xeno_rt_amd.config import (ConfigError, LlamaConfig, architecture, load_config, parse_config,
                                register_architecture, registered_architectures, save_config)


@pytest.mark.parametrize("name", ["llama", "qwen3"])
def test_tiny_configs_round_trip(name, tmp_path):
    config = parse_config(TINY[name])
    save_config(config, str(tmp_path))
    assert load_config(str(tmp_path)) == config
    assert parse_config(config.to_dict()) == config


def test_every_size_and_option_differs_between_the_tiny_configs():
    a, b = parse_config(TINY["llama"]), parse_config(TINY["qwen3"])
    for field in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                  "num_key_value_heads", "head_dim", "rms_norm_eps", "rope_theta", "max_position_embeddings",
                  "tie_word_embeddings", "qk_norm", "eos_token_ids", "bos_token_id"):
        assert getattr(a, field) != getattr(b, field), field
    assert b.head_dim != b.hidden_size // b.num_attention_heads      # decoupled head size
    assert b.q_width == 192 and b.kv_width == 96 and a.q_width == 64 and a.kv_width == 32


def test_defaults_of_absent_keys_are_the_references():
    raw = {k: v for k, v in TINY["llama"].items()
           if k not in ("num_key_value_heads", "rms_norm_eps", "rope_theta", "eos_token_id", "bos_token_id")}
    config = parse_config(raw)
    assert config.num_key_value_heads == config.num_attention_heads       # llama.rs:68-70
    assert config.head_dim == 16                                          # llama.rs:125-128
    assert config.rms_norm_eps == 1e-5 and config.rope_theta == 10000.0   # llama.rs:95-102
    assert config.eos_token_ids == () and config.bos_token_id is None
    assert config.rope_dim == config.head_dim


def test_rotary_base_inside_rope_parameters_is_read_not_ignored():
    raw = {k: v for k, v in TINY["qwen3"].items() if k not in ("rope_theta", "rope_scaling", "partial_rotary_factor")}
    raw["rope_parameters"] = {"rope_theta": 1000000.0, "rope_type": "linear", "factor": 4.0, "partial_rotary_factor": 0.5}
    assert parse_config(raw).rope_theta == 1000000.0
    assert parse_config(raw) == parse_config(TINY["qwen3"])
    raw = {k: v for k, v in TINY["llama"].items() if k != "rope_theta"}
    raw["rope_parameters"] = {"rope_theta": 10000.0, "rope_type": "default"}
    assert parse_config(raw) == parse_config(TINY["llama"])


def test_the_rotation_s_options():
    """How many dims of a head are rotated and what multiplies a position (llama.rs:92-94, 103-106): a share of the
    head and a linear rule whose factor divides the positions."""
    plain = parse_config(TINY["llama"])
    assert plain.rope_dim == plain.head_dim == 16 and plain.rope_scale == 1.0
    assert "rope_scaling" not in plain.to_dict() and "partial_rotary_factor" not in plain.to_dict()
    both = parse_config(TINY["qwen3"])
    assert both.head_dim == 32 and both.rope_dim == 16 and both.rope_scale == 0.25
    assert parse_config(both.to_dict()) == both
    older = parse_config(dict(TINY["llama"], rope_scaling={"type": "linear", "factor": 2}))     # the older spelling of the key
    assert older.rope_scale == 0.5 and older.rope_dim == 16
    assert parse_config(dict(TINY["llama"], rope_scaling={"rope_type": "default"})) == plain
    assert parse_config(dict(TINY["llama"], partial_rotary_factor=1.0, rope_scaling=None)) == plain


def test_written_config_names_its_model_type(tmp_path):
    for name, model_type in (("llama", "llama"), ("qwen3", "qwen3")):
        assert parse_config(TINY[name]).to_dict()["model_type"] == model_type


def test_eos_may_be_a_number_or_a_list():
    assert parse_config(TINY["llama"]).eos_token_ids == (1,)
    assert parse_config(TINY["qwen3"]).eos_token_ids == (2, 5)


@pytest.mark.parametrize("change, text", [
    ({"architectures": ["MambaForCausalLM"]}, "unsupported architecture"),
    ({"architectures": []}, "non-empty"),
    ({"hidden_size": None}, "hidden_size"),
    ({"num_hidden_layers": 0}, "num_hidden_layers"),
    ({"num_attention_heads": 5}, "not divisible"),
    ({"num_key_value_heads": 3}, "not divisible"),
    ({"num_key_value_heads": 0}, "non-zero"),
    ({"head_dim": 15}, "even"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "rope_type"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0}}, "not supported"),
    ({"rope_scaling": {"type": "linear"}}, "factor"),
    ({"rope_scaling": {"type": "linear", "factor": 0}}, "factor"),
    ({"rope_scaling": {"factor": 2.0}}, "without a rule"),
    ({"rope_scaling": {"type": "linear", "factor": 2.0}, "rope_parameters": {"rope_type": "linear", "factor": 4.0}}, "disagree"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"attention_bias": True}, "attention_bias"),
    ({"mlp_bias": True}, "mlp_bias"),
    ({"eos_token_id": 9999}, "outside the vocabulary"),
    ({"rms_norm_eps": 0.0}, "rms_norm_eps"),
    ({"vocab_size": "many"}, "vocab_size"),
    ({"model_type": "qwen3"}, "model_type"),
    ({"rope_parameters": {"rope_theta": 10000.0, "rope_type": "yarn"}}, "rope_type"),
    ({"rope_parameters": {"rope_theta": 10000.0, "factor": 4.0}}, "without a rule"),
    ({"rope_parameters": {"rope_theta": 10000.0, "beta_fast": 32}}, "not supported"),
    ({"rope_parameters": {"rope_theta": 500000.0}}, "disagree"),
    ({"partial_rotary_factor": 0.2}, "rotated dims"),          # 3.2 of 16 dims: three
    ({"partial_rotary_factor": 1.5}, "partial_rotary_factor"),
    ({"partial_rotary_factor": 0.01}, "rotated dims"),
    ({"partial_rotary_factor": 0.5, "rope_parameters": {"partial_rotary_factor": 0.25}}, "disagree"),
])
def test_bad_configs_are_refused(change, text):
    with pytest.raises(ConfigError, match=text):
        parse_config(dict(TINY["llama"], **change))


def test_missing_and_broken_files(tmp_path):
    with pytest.raises(ConfigError, match="no config.json"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="invalid JSON"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps([1, 2]))
    with pytest.raises(ConfigError, match="JSON object"):
        load_config(str(tmp_path))


def test_registry_maps_names_to_builders():
    assert {"LlamaForCausalLM", "Qwen3ForCausalLM"} <= set(registered_architectures())
    llama, qwen = architecture("LlamaForCausalLM"), architecture("Qwen3ForCausalLM")
    assert llama.config_class is LlamaConfig and qwen.config_class is LlamaConfig
    spec = qwen.build(parse_config(TINY["qwen3"]))
    assert len(spec.layers) == 3 and spec.head.tied_to is spec.embedding
    assert spec.layers[0].mixer.qk_norm and not llama.build(parse_config(TINY["llama"])).layers[0].mixer.qk_norm
    assert [c.layer for c in spec.schedule] == [0, 1, 2]

    class Other:
        @classmethod
        def from_dict(cls, raw):
            return "parsed"
    register_architecture("OtherForCausalLM", Other, lambda config: None)
    assert parse_config({"architectures": ["OtherForCausalLM"]}) == "parsed"


def test_model_description_names_the_checkpoint_tensors():
    spec = architecture("Qwen3ForCausalLM").build(parse_config(TINY["qwen3"]))
    names = spec.weight_specs()
    assert names["model.layers.2.self_attn.q_proj.weight"].shape == (192, 96)
    assert names["model.layers.0.self_attn.k_norm.weight"].shape == (32,)
    assert names["model.layers.1.mlp.down_proj.weight"].shape == (96, 256)
    assert "lm_head.weight" not in names and spec.ignored_names() == ["lm_head.weight"]
    llama = architecture("LlamaForCausalLM").build(parse_config(TINY["llama"]))
    assert llama.weight_specs()["lm_head.weight"].shape == (256, 64)
    assert not any("q_norm" in name for name in llama.weight_specs())
