"""Configuration and registry (no GPU)."""
import json

import pytest

import gpullama3_java_amd as g
from gpullama3_java_amd.config import ConfigError, Llama3RopeScaling, config_from_dict, load_config
from tiny import TINY_A, TINY_B, TINY_C


def test_reads_every_size_from_the_keys():
    c = config_from_dict(TINY_B)
    assert (c.hidden_size, c.intermediate_size, c.num_hidden_layers) == (96, 320, 3)
    assert (c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (3, 1, 32)
    assert (c.vocab_size, c.max_position_embeddings) == (384, 256)
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 500000.0 and not c.tie_word_embeddings
    assert c.rope_scaling == Llama3RopeScaling(8.0, 1.0, 4.0, 64)
    assert c.kv_dim == 32 and c.kv_mul == 3 and c.rope_pairing == "half"


def test_defaults_follow_the_reference():
    d = {k: v for k, v in TINY_A.items() if k not in ("num_key_value_heads", "head_dim", "rms_norm_eps",
                                                       "rope_theta", "rope_scaling", "rope_pairing",
                                                       "tie_word_embeddings")}
    c = config_from_dict(d)
    assert c.num_key_value_heads == c.num_attention_heads == 4      # LlamaModelLoader.java:39-41
    assert c.head_dim == 16                                           # LlamaConfiguration.java:27-29
    assert c.rms_norm_eps == 1e-5 and c.rope_theta == 10000.0         # LlamaModelLoader.java:45-46
    assert c.rope_scaling is None and not c.tie_word_embeddings


def test_head_dim_need_not_be_hidden_over_heads():
    c = config_from_dict(TINY_C)
    assert c.head_dim * c.num_attention_heads != c.hidden_size
    spec = c.model_spec()
    assert spec.layers[0].mixer.head_dim == 48 and spec.layers[0].mixer.hidden == 112


@pytest.mark.parametrize("change, word", [
    ({"architectures": ["MistralForCausalLM"]}, "unknown architecture"),
    ({"architectures": []}, "architectures"),
    ({"hidden_size": None}, "hidden_size"),
    ({"vocab_size": -5}, "vocab_size"),
    ({"num_hidden_layers": 2.5}, "num_hidden_layers"),
    ({"num_key_value_heads": 3}, "not a multiple"),
    ({"head_dim": 15}, "odd"),
    ({"attention_bias": True}, "attention_bias"),
    ({"mlp_bias": True}, "mlp_bias"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2}}, "rope_type"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 2}}, "low_freq_factor"),
    ({"rope_pairing": "both"}, "rope_pairing"),
    ({"rms_norm_eps": 0}, "positive"),
])
def test_errors_name_the_key(change, word):
    with pytest.raises(ConfigError) as e:
        config_from_dict({**TINY_A, **change})
    assert word in str(e.value)


def test_unknown_architecture_lists_the_registered():
    with pytest.raises(ConfigError) as e:
        config_from_dict({**TINY_A, "architectures": ["Nope"]})
    assert "LlamaForCausalLM" in str(e.value)


def test_round_trip_and_folder(tmp_path):
    c = config_from_dict(TINY_B)
    assert config_from_dict(c.to_dict()) == c
    (tmp_path / "config.json").write_text(json.dumps(c.to_dict()))
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": [7, 9]}))
    assert load_config(str(tmp_path)).stop_ids == (7, 9)
    with pytest.raises(FileNotFoundError):
        load_config(str(tmp_path / "nothing"))


def test_context_length_override():
    c = config_from_dict(TINY_B)
    assert c.with_context_length(-1) is c                       # negative keeps the model's
    assert c.with_context_length(100).max_position_embeddings == 100
    assert c.with_context_length(10**6).max_position_embeddings == 256


def test_model_spec_is_layer_by_layer_data():
    spec = config_from_dict(TINY_A).model_spec()
    assert len(spec.layers) == 2 and [r.layer for r in spec.run_order] == [0, 1]
    assert all(r.reads is None for r in spec.run_order)
    b = spec.layers[1]
    assert b.kind == "prenorm" and b.mixer.kind == "attention" and b.ffn.kind == "gated"
    assert b.mixer.names["q"] == "model.layers.1.self_attn.q_proj.weight"
    assert b.mixer.position.pairing == "adjacent" and b.mixer.position.theta == 10000.0
    assert b.mixer_norm.eps == 1e-5 and spec.tie_embeddings and spec.head_name is None
    assert config_from_dict(TINY_B).model_spec().head_name == "lm_head.weight"


def test_registering_another_architecture():
    class Other:
        @classmethod
        def from_dict(cls, d):
            return cls()
    g.register_architecture("OtherForCausalLM", Other)
    assert isinstance(config_from_dict({"architectures": ["OtherForCausalLM"]}), Other)
    assert "OtherForCausalLM" in g.registered_architectures()
