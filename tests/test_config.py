"""Typed configuration and architecture registry (CPU)."""

import json

import pytest

from llm_runtime_study_amd.config import (Qwen3Config, config_from_dict, load_config, registered_architectures, spec_for)
from llm_runtime_study_amd.errors import ConfigError
from tests.helpers import TINY_A, TINY_B


def qwen3_06b():
    # the sizes of the reference's test configuration (reference tests/test_config.py valid_config)
    return {
        "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": 151936, "hidden_size": 1024,
        "intermediate_size": 3072, "num_hidden_layers": 28, "num_attention_heads": 16, "num_key_value_heads": 8,
        "head_dim": 128, "max_position_embeddings": 40960, "rms_norm_eps": 1e-6, "rope_theta": 1000000,
        "hidden_act": "silu", "attention_bias": False, "attention_dropout": 0.0, "tie_word_embeddings": True,
        "torch_dtype": "bfloat16", "bos_token_id": 151643, "eos_token_id": 151645,
    }


def test_derived_sizes_do_not_assume_hidden_per_head():
    # reference tests/test_config.py:162-175
    config = Qwen3Config.from_dict(qwen3_06b())
    assert (config.query_projection_size, config.kv_projection_size, config.queries_per_kv_head) == (2048, 1024, 2)
    assert config.kv_cache_bytes(4096, dtype="float16") == 28 * 2 * 1 * 8 * 4096 * 128 * 2 == 469_762_048
    assert config.rope_theta == 1e6 and isinstance(config.rope_theta, float)


def test_eos_list_and_context_limit():
    raw = qwen3_06b()
    raw["eos_token_id"] = [151645, 151643]
    assert Qwen3Config.from_dict(raw).eos_token_ids == (151645, 151643)
    with pytest.raises(ConfigError, match="exceeds the model limit"):
        Qwen3Config.from_dict(qwen3_06b()).kv_cache_bytes(40961)
    with pytest.raises(ConfigError, match="must be positive"):
        Qwen3Config.from_dict(qwen3_06b()).validate_context_length(0)


@pytest.mark.parametrize("field,bad,message", [
    ("num_key_value_heads", 6, "divisible"),
    ("head_dim", 127, "even for rotary embeddings"),
    ("rms_norm_eps", "small", "int or float"),
    ("bos_token_id", 151936, "within vocabulary"),
    ("model_type", "llama", "unsupported model_type"),
    ("vocab_size", True, "must be int, got bool"),
    ("hidden_size", 0, "must be positive"),
    ("hidden_act", "gelu", "unsupported hidden_act"),
    ("torch_dtype", "int8", "unsupported torch_dtype"),
    ("attention_bias", 1, "must be boolean"),
    ("eos_token_id", [], "non-empty integer list"),
    ("rope_theta", -1.0, "rope_theta must be positive"),
])
def test_rejects_invalid_fields(field, bad, message):
    raw = qwen3_06b()
    raw[field] = bad
    with pytest.raises(ConfigError, match=message):
        Qwen3Config.from_dict(raw)


def test_missing_field_is_named():
    raw = qwen3_06b()
    del raw["head_dim"]
    with pytest.raises(ConfigError, match="missing required configuration field: head_dim"):
        Qwen3Config.from_dict(raw)


def test_registry_dispatch_and_file_errors(tmp_path):
    assert "Qwen3ForCausalLM" in registered_architectures()
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    config = load_config(tmp_path)
    assert isinstance(config, Qwen3Config) and config.hidden_size == 96
    unknown = dict(TINY_B, architectures=["SomethingElse"])
    with pytest.raises(ConfigError, match="no model is registered for architecture 'SomethingElse'.*Qwen3ForCausalLM"):
        config_from_dict(unknown)
    with pytest.raises(ConfigError, match="model directory does not exist"):
        load_config(tmp_path / "nope")
    (tmp_path / "empty").mkdir()
    with pytest.raises(ConfigError, match="model configuration does not exist"):
        load_config(tmp_path / "empty")
    (tmp_path / "empty" / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="invalid JSON"):
        load_config(tmp_path / "empty")
    (tmp_path / "empty" / "config.json").write_text("[1]")
    with pytest.raises(ConfigError, match="root must be an object"):
        load_config(tmp_path / "empty")


def test_config_round_trips_through_json():
    for raw in (TINY_A, TINY_B):
        config = config_from_dict(raw)
        assert config_from_dict(json.loads(json.dumps(config.to_json_dict()))) == config


def test_spec_carries_every_constant_of_the_configuration():
    """No size stands in code: the parts' parameters all come from the configuration."""
    for raw in (TINY_A, TINY_B):
        config = config_from_dict(raw)
        spec = spec_for(config)
        assert len(spec.layers) == config.num_hidden_layers == len(spec.schedule)
        assert spec.tie_head == config.tie_word_embeddings and spec.vocab_size == config.vocab_size
        mixer = spec.layers[0].params["mixer"].params
        assert (mixer["num_heads"], mixer["num_kv_heads"], mixer["head_dim"]) == (
            config.num_attention_heads, config.num_key_value_heads, config.head_dim)
        assert mixer["qk_norm_eps"] == config.rms_norm_eps and mixer["bias"] == config.attention_bias
        assert mixer["position"].params == {"rotary_dim": config.head_dim, "theta": config.rope_theta}
        assert spec.layers[0].params["feed_forward"].params["intermediate_size"] == config.intermediate_size
        assert spec.final_norm.params == {"size": config.hidden_size, "eps": config.rms_norm_eps}
