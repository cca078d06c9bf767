"""Typed configuration and the architecture registry."""
import json
import os
import warnings

import pytest

import inferllm_amd as I
from inferllm_amd.config import ConfigError, ModelSpec
from tiny import CONFIGS, TINY_A, TINY_B


def test_llama_config_reads_its_keys_and_defaults():
    c = I.config_from_dict({"architectures": ["LlamaForCausalLM"], "hidden_size": 64,
                            "intermediate_size": 172, "num_hidden_layers": 2,
                            "num_attention_heads": 4, "vocab_size": 256})
    assert c.num_key_value_heads == 4 and c.head_dim == 16
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 10000.0 and c.max_position_embeddings == 2048
    assert c.eos_token_id == [2] and c.bos_token_id == 1 and not c.tie_word_embeddings
    b = I.config_from_dict(TINY_B)
    assert (b.num_key_value_heads, b.head_dim, b.rope_theta, b.rms_norm_eps) == (2, 24, 500000.0, 1e-5)
    assert b.eos_token_id == [2, 3]


def test_spec_carries_every_constant_of_the_config():
    for name, cfg in CONFIGS.items():
        c = I.config_from_dict(cfg)
        spec = c.to_spec()
        assert isinstance(spec, ModelSpec) and len(spec.layers) == cfg["num_hidden_layers"]
        L = spec.layers[-1]
        assert L.mixer.params["num_kv_heads"] == c.num_key_value_heads
        assert L.mixer.params["head_dim"] == c.head_dim
        assert L.mixer_norm.params["eps"] == cfg["rms_norm_eps"] == spec.final_norm.params["eps"]
        assert L.position.params["theta"] == cfg["rope_theta"]
        assert L.position.params["max_positions"] == cfg["max_position_embeddings"]
        assert L.feed_forward.params["intermediate_size"] == cfg["intermediate_size"]
        assert [e.layer for e in spec.schedule] == list(range(len(spec.layers)))
        assert spec.eos_token_ids == c.eos_token_id


def test_round_trip_through_a_folder(tmp_path):
    c = I.config_from_dict(TINY_B)
    (tmp_path / "config.json").write_text(json.dumps(c.to_dict()))
    assert I.load_config(str(tmp_path)) == c


@pytest.mark.parametrize("change,match", [
    ({"architectures": ["GPT2LMHeadModel"]}, "unsupported architecture"),
    ({"architectures": []}, "architectures"),
    ({"hidden_size": None}, "positive integer"),
    ({"num_attention_heads": 3}, "not a multiple"),
    ({"num_key_value_heads": 3}, "not a multiple"),
    ({"head_dim": 15}, "even"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"attention_bias": True}, "bias"),
    ({"rope_scaling": {"type": "linear", "factor": 2.0}}, "rope_scaling"),
    ({"rms_norm_eps": 0.0}, "rms_norm_eps"),
    ({"eos_token_id": 999}, "outside the vocabulary"),
    ({"vocab_size": -1}, "positive integer"),
])
def test_bad_configs_are_refused_with_a_reason(change, match):
    d = dict(TINY_A)
    d.update(change)
    with pytest.raises(ConfigError, match=match):
        I.config_from_dict(d)


def test_missing_required_keys_are_listed():
    d = dict(TINY_A)
    del d["intermediate_size"], d["vocab_size"]
    with pytest.raises(ConfigError) as e:
        I.config_from_dict(d)
    assert "intermediate_size" in str(e.value) and "vocab_size" in str(e.value)


def test_unknown_keys_warn(tmp_path):
    d = dict(TINY_A, some_new_option=3)
    with pytest.warns(UserWarning, match="some_new_option"):
        I.config_from_dict(d)


def test_no_config_json(tmp_path):
    with pytest.raises(ConfigError, match="config.json"):
        I.load_config(str(tmp_path))


def test_registry_takes_another_architecture():
    from inferllm_amd.config import register_architecture, registered_architectures

    @register_architecture("ToyForTests")
    class ToyConfig:
        @classmethod
        def from_dict(cls, d):
            return cls()

    assert "ToyForTests" in registered_architectures()
    assert isinstance(I.config_from_dict({"architectures": ["ToyForTests"]}), ToyConfig)
