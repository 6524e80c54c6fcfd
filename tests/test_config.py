"""Configuration and registry (no GPU).  Defaults and required keys are the
reference's (models/config.go:107-119)."""

import json

import pytest

import tiny
from kllm_amd.config import (ConfigError, LlamaConfig, config_from_dict, load_config,
                             register_architecture, registered_architectures,
                             unregister_architecture)

MINIMAL = {"architectures": ["LlamaForCausalLM"], "hidden_size": 64, "num_hidden_layers": 2,
           "num_attention_heads": 4, "vocab_size": 256, "intermediate_size": 176}


def test_defaults_are_the_references():
    c = config_from_dict(MINIMAL)
    assert isinstance(c, LlamaConfig)
    assert c.num_key_value_heads == 4          # defaults to the head count
    assert c.head_dim == 16                    # hidden / heads
    assert c.rope_theta == 10000.0 and c.rms_norm_eps == 1e-6
    assert c.eos_token_ids == () and c.tie_word_embeddings is False
    assert c.max_position_embeddings is None
    assert c.q_dim == 64 and c.kv_dim == 64


@pytest.mark.parametrize("name", ["A", "B", "C", "D", "R"])
def test_every_size_comes_from_config_json(name, tmp_path):
    raw = tiny.CONFIGS[name]
    (tmp_path / "config.json").write_text(json.dumps(raw))
    c = load_config(str(tmp_path))
    assert c.hidden_size == raw["hidden_size"] and c.head_dim == raw["head_dim"]
    assert c.num_key_value_heads == raw.get("num_key_value_heads", raw["num_attention_heads"])
    assert c.rope_theta == raw["rope_theta"] and c.rms_norm_eps == raw["rms_norm_eps"]
    assert c.tie_word_embeddings == raw["tie_word_embeddings"]
    assert c.max_position_embeddings == raw["max_position_embeddings"]
    again = config_from_dict(c.to_dict())
    assert again == c


def test_head_dim_may_differ_from_hidden_over_heads():
    c = config_from_dict(dict(MINIMAL, head_dim=48))
    assert c.head_dim == 48 and c.q_dim == 192


@pytest.mark.parametrize("key", ["hidden_size", "num_hidden_layers", "num_attention_heads",
                                 "vocab_size", "intermediate_size"])
def test_required_keys(key):
    raw = dict(MINIMAL)
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        config_from_dict(raw)
    with pytest.raises(ConfigError, match=key):
        config_from_dict(dict(MINIMAL, **{key: 0}))


def test_eos_may_be_int_list_or_absent():
    assert config_from_dict(dict(MINIMAL, eos_token_id=2)).eos_token_ids == (2,)
    assert config_from_dict(dict(MINIMAL, eos_token_id=[128001, 128009])).eos_token_ids == (128001, 128009)
    assert config_from_dict(dict(MINIMAL, eos_token_id=-1)).eos_token_ids == ()
    assert config_from_dict(dict(MINIMAL, eos_token_id=None)).eos_token_ids == ()
    with pytest.raises(ConfigError):
        config_from_dict(dict(MINIMAL, eos_token_id="</s>"))


def test_rope_parameters_block():
    # transformers >= 5 nests the base (models/config.go:56-99)
    c = config_from_dict(dict(MINIMAL, rope_parameters={"rope_theta": 500000.0, "rope_type": "default"}))
    assert c.rope_theta == 500000.0
    with pytest.raises(ConfigError, match="rope"):
        config_from_dict(dict(MINIMAL, rope_parameters={"rope_theta": 1e4, "rope_type": "llama3"}))


@pytest.mark.parametrize("extra,word", [
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8.0}}, "rope_scaling"),
    ({"rope_scaling": {"type": "linear", "factor": 2.0}}, "rope_scaling"),
    ({"attention_bias": True}, "attention_bias"),
    ({"mlp_bias": True}, "mlp_bias"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"num_key_value_heads": 3}, "num_key_value_heads"),
    ({"head_dim": 15}, "head_dim"),
    ({"hidden_size": 66}, "head_dim"),
])
def test_what_would_change_the_result_is_refused(extra, word):
    with pytest.raises(ConfigError, match=word):
        config_from_dict(dict(MINIMAL, **extra))


def test_harmless_values_are_accepted():
    config_from_dict(dict(MINIMAL, rope_scaling=None, attention_bias=False, mlp_bias=False,
                          hidden_act="silu", pretraining_tp=1, torch_dtype="bfloat16",
                          use_cache=True, initializer_range=0.02, transformers_version="4.40"))


def test_registry_names_what_it_knows():
    assert "LlamaForCausalLM" in registered_architectures()
    with pytest.raises(ConfigError) as e:
        config_from_dict(dict(MINIMAL, architectures=["MixtralForCausalLM"]))
    assert "MixtralForCausalLM" in str(e.value) and "LlamaForCausalLM" in str(e.value)
    raw = dict(MINIMAL)
    del raw["architectures"]
    with pytest.raises(ConfigError):
        config_from_dict(raw)
    assert isinstance(config_from_dict(dict(raw, model_type="llama")), LlamaConfig)


def test_another_architecture_can_be_registered():
    calls = []

    def build(cfg):
        calls.append(cfg)
        return "spec"
    register_architecture("ToyForCausalLM", LlamaConfig, build)
    try:
        from kllm_amd.config import resolve_architecture
        raw = dict(MINIMAL, architectures=["ToyForCausalLM"])
        arch = resolve_architecture(raw)
        assert arch.build(config_from_dict(raw)) == "spec" and len(calls) == 1
    finally:
        unregister_architecture("ToyForCausalLM")
    assert "ToyForCausalLM" not in registered_architectures()


def test_config_file_errors(tmp_path):
    with pytest.raises(ConfigError, match="no such file"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="JSON"):
        load_config(str(tmp_path))


def test_model_spec_takes_every_constant_from_the_config():
    from kllm_amd.config import resolve_architecture
    raw = tiny.CONFIGS["B"]
    spec = resolve_architecture(raw).build(config_from_dict(raw))
    assert len(spec.layers) == 3 and [r.layer for r in spec.schedule] == [0, 1, 2]
    m = spec.layers[1].mixer.params
    assert (m["heads"], m["kv_heads"], m["head_dim"]) == (3, 1, 32)
    assert m["position"].params == {"head_dim": 32, "theta": 500000.0}
    assert spec.layers[0].norm_mixer.params["eps"] == 1e-6
    assert spec.layers[2].feed_forward.params["intermediate"] == 256
    assert spec.head.prefix == "model.embed_tokens"          # tied
    specA = resolve_architecture(tiny.CONFIGS["A"]).build(config_from_dict(tiny.CONFIGS["A"]))
    assert specA.head.prefix == "lm_head" and specA.final_norm.params["eps"] == 1e-5
