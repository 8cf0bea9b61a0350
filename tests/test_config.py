"""Configuration and registry: config.json's own keys, defaults, validation, the one table of architectures."""
import json
import os

import pytest

from helpers import TINY_A, TINY_B, TINY_C

from lmsf_amd.config import (ConfigError, LlamaConfig, RopeScaling, get_architecture, load_model_config,
                             register_architecture, registered_architectures, resolve_architecture,
                             unregister_architecture)


def test_every_size_comes_from_the_keys():
    a, b = LlamaConfig.from_dict(TINY_A), LlamaConfig.from_dict(TINY_B)
    assert (a.hidden_size, a.num_attention_heads, a.num_key_value_heads, a.head_dim) == (64, 4, 2, 16)   # head_dim derived
    assert (b.hidden_size, b.num_attention_heads, b.num_key_value_heads, b.head_dim) == (128, 8, 1, 32)  # explicit
    assert (a.intermediate_size, b.intermediate_size, a.vocab_size, b.vocab_size) == (176, 352, 256, 1000)
    assert (a.rms_norm_eps, b.rms_norm_eps, a.rope_theta, b.rope_theta) == (1e-5, 1e-6, 10000.0, 500000.0)
    assert a.rope_scaling is None and b.rope_scaling == RopeScaling("llama3", 8.0, 1.0, 4.0, 64)
    assert (a.tie_word_embeddings, b.tie_word_embeddings, a.attention_bias, b.attention_bias) == (True, False, False, True)
    assert a.eos_token_ids == (2,) and b.eos_token_ids == (7, 9)
    assert LlamaConfig.from_dict(TINY_C).mlp_bias is True
    assert (a.max_position_embeddings, b.max_position_embeddings, a.num_hidden_layers, b.num_hidden_layers) == (128, 512, 2, 3)


def test_defaults_of_optional_keys():
    d = {k: v for k, v in TINY_A.items() if k not in ("num_key_value_heads", "rope_theta", "tie_word_embeddings",
                                                       "attention_bias", "rope_scaling", "bos_token_id",
                                                       "eos_token_id", "hidden_act", "torch_dtype")}
    c = LlamaConfig.from_dict(d)
    assert c.num_key_value_heads == c.num_attention_heads            # core/src/model_executor/models/model.rs:24-26
    assert c.rope_theta == 10000.0                                   # llama/config.rs:28-30
    assert (c.tie_word_embeddings, c.attention_bias, c.mlp_bias, c.rope_scaling) == (False, False, False, None)
    assert c.eos_token_ids == () and c.bos_token_id is None and c.torch_dtype == "bfloat16"


def test_round_trip_through_to_dict():
    for d in (TINY_A, TINY_B, TINY_C):
        c = LlamaConfig.from_dict(d)
        assert LlamaConfig.from_dict(json.loads(json.dumps(c.to_dict()))) == c


@pytest.mark.parametrize("change,word", [
    ({"hidden_size": None}, "hidden_size"),
    ({"rms_norm_eps": None}, "rms_norm_eps"),
    ({"vocab_size": "many"}, "vocab_size"),
    ({"num_hidden_layers": 2.5}, "num_hidden_layers"),
    ({"num_key_value_heads": 3}, "multiple of num_key_value_heads"),
    ({"hidden_size": 66}, "no head_dim"),
    ({"head_dim": 15}, "even"),
    ({"rms_norm_eps": 0.0}, "rms_norm_eps"),
    ({"rope_theta": -1.0}, "rope_theta"),
    ({"hidden_act": "relu"}, "hidden_act"),
    ({"torch_dtype": "int8"}, "torch_dtype"),
    ({"eos_token_id": 256}, "eos_token_id"),
    ({"tie_word_embeddings": "yes"}, "tie_word_embeddings"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "rope_type"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8.0}}, "low_freq_factor"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 4.0, "high_freq_factor": 4.0,
                       "original_max_position_embeddings": 64}}, "high_freq_factor"),
    ({"rope_scaling": 3}, "rope_scaling"),
])
def test_bad_values_name_the_key(change, word):
    d = dict(TINY_A)
    d.update(change)
    with pytest.raises(ConfigError, match=word):
        LlamaConfig.from_dict(d)


def test_rope_scaling_spellings():
    assert RopeScaling.from_dict(None) is None
    assert RopeScaling.from_dict({"rope_type": "default"}) == RopeScaling()
    old = RopeScaling.from_dict({"type": "llama3", "factor": 2, "low_freq_factor": 1, "high_freq_factor": 4,
                                 "original_max_position_embeddings": 8192})
    assert old.rope_type == "llama3" and old.factor == 2.0


def test_registry_by_architecture_then_model_type(tmp_path):
    assert "LlamaForCausalLM" in registered_architectures()
    arch = resolve_architecture({"architectures": ["LlamaForCausalLM"]})
    assert arch is get_architecture("LlamaForCausalLM") and arch.config_class is LlamaConfig
    assert resolve_architecture({"model_type": "LLaMA"}) is arch         # case-insensitive, model_factory.rs:44-50
    with pytest.raises(ConfigError, match="registered: .*LlamaForCausalLM"):
        resolve_architecture({"architectures": ["GemmaForCausalLM"]})
    with pytest.raises(ConfigError, match="model_type"):
        resolve_architecture({"model_type": "opt"})
    with pytest.raises(ConfigError, match="neither"):
        resolve_architecture({})
    folder = str(tmp_path)
    with pytest.raises(ConfigError, match="no config.json"):
        load_model_config(folder)
    with open(os.path.join(folder, "config.json"), "w") as f:
        f.write("{not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        load_model_config(folder)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(TINY_B, f)
    got_arch, cfg = load_model_config(folder)
    assert got_arch is arch and cfg == LlamaConfig.from_dict(TINY_B)


def test_registering_another_architecture_needs_one_call():
    class ToyConfig(LlamaConfig):
        ARCHITECTURE = "ToyForCausalLM"
        MODEL_TYPE = "toy"

    try:
        register_architecture("ToyForCausalLM", "toy", ToyConfig, get_architecture("LlamaForCausalLM").build_spec)
        with pytest.raises(ValueError, match="already registered"):
            register_architecture("ToyForCausalLM", "toy", ToyConfig, None)
        cfg = resolve_architecture({"model_type": "toy"}).config_class.from_dict(TINY_A)
        assert cfg.architecture == "ToyForCausalLM" and cfg.to_dict()["architectures"] == ["ToyForCausalLM"]
    finally:
        unregister_architecture("ToyForCausalLM")
    assert "ToyForCausalLM" not in registered_architectures()


def test_the_configuration_is_read_and_checked_by_the_host_library(tmp_path):
    """from_dict hands the keys to the C++ reader (csrc/host/llama_config.cc) and takes back what it read: null
    counts as absent, an integer written as 2.0 is one, text is read with its escapes, and what ``replace`` makes is
    checked by the same code."""
    from lmsf_amd.config.model_config import replace
    d = dict(TINY_A, num_hidden_layers=2.0, rope_theta=None, hidden_act="silu")
    c = LlamaConfig.from_dict(d)
    assert c.num_hidden_layers == 2 and isinstance(c.num_hidden_layers, int) and c.rope_theta == 10000.0
    folder = str(tmp_path)
    with open(os.path.join(folder, "config.json"), "w") as f:
        f.write(json.dumps(dict(TINY_B, hidden_act="silu")).replace('"silu"', '"si\\u006cu"').replace(", ", " ,\n\t"))
    assert load_model_config(folder)[1] == LlamaConfig.from_dict(TINY_B)
    with pytest.raises(ConfigError, match="at most 16"):
        LlamaConfig.from_dict(dict(TINY_A, eos_token_id=list(range(17))))
    with pytest.raises(ConfigError, match="eos_token_id"):
        LlamaConfig.from_dict(dict(TINY_A, eos_token_id=[1, "two"]))
    with pytest.raises(ConfigError, match="multiple of num_key_value_heads"):
        replace(c, num_key_value_heads=3)
    with pytest.raises(ConfigError, match="JSON"):
        LlamaConfig.from_dict(dict(TINY_A, hidden_size=float("inf")))
    assert replace(c, num_key_value_heads=4).num_key_value_heads == 4
