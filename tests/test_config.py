"""Configuration parsing and the architecture registry (no GPU)."""
import json

import pytest

from llmengine.config import (ConfigError, LlamaConfig, known_architectures, load_config, parse_config,
                              register_architecture, resolve)
from tiny_models import TINY_A, TINY_B


def test_fields_and_defaults():
    c = parse_config(TINY_B)
    assert isinstance(c, LlamaConfig)
    assert (c.hidden_size, c.intermediate_size, c.num_hidden_layers) == (96, 256, 3)
    assert (c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (3, 1, 32)
    assert (c.vocab_size, c.max_position_embeddings, c.rms_norm_eps, c.rope_theta) == (384, 256, 1e-6, 500000.0)
    s = c.rope_scaling
    assert (s.factor, s.low_freq_factor, s.high_freq_factor, s.original_max_position_embeddings) == (32.0, 1.0, 4.0, 64)
    assert not c.tie_word_embeddings and c.eos_token_ids == ()
    assert c.max_pos == 256                              # not capped at the scaling's original length
    minimal = {"architectures": ["LlamaForCausalLM"], "hidden_size": 64, "intermediate_size": 8,
               "num_hidden_layers": 1, "num_attention_heads": 4, "vocab_size": 10, "max_position_embeddings": 16}
    m = parse_config(minimal)                            # defaults of src/weights.cpp:59-79
    assert (m.num_key_value_heads, m.head_dim, m.rms_norm_eps, m.rope_theta) == (4, 16, 1e-5, 10000.0)
    assert m.rope_scaling is None and not m.tie_word_embeddings


def test_round_trip():
    for cfg in (TINY_A, TINY_B):
        c = parse_config(cfg)
        assert parse_config(c.to_dict()) == c


def test_rope_parameters_block_wins():
    cfg = dict(TINY_A, rope_scaling={"rope_type": "llama3", "factor": 2.0},
               rope_parameters={"rope_theta": 123.0, "rope_type": "llama3", "factor": 8.0,
                                "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                "original_max_position_embeddings": 32})
    c = parse_config(cfg)
    assert c.rope_theta == 123.0 and c.rope_scaling.factor == 8.0
    d = parse_config(dict(TINY_A, rope_parameters={"rope_theta": 5.0, "rope_type": "default"}))
    assert d.rope_theta == 5.0 and d.rope_scaling is None


def test_eos_union(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(dict(TINY_A, eos_token_id=2)))
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": [1, 2, 3]}))
    assert load_config(str(tmp_path)).eos_token_ids == (1, 2, 3)


@pytest.mark.parametrize("change,needle", [
    ({"hidden_size": None}, "hidden_size"),
    ({"num_hidden_layers": 0}, "num_hidden_layers"),
    ({"vocab_size": "big"}, "vocab_size"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"head_dim": 15}, "even"),
    ({"attention_bias": True}, "attention_bias"),
    ({"mlp_bias": True}, "mlp_bias"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "yarn"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 0}}, "factor"),
    ({"architectures": ["MysteryForCausalLM"]}, "unknown architecture"),
    ({"architectures": []}, "architectures"),
])
def test_refusals_name_the_key(change, needle):
    cfg = {k: v for k, v in dict(TINY_A, **change).items() if v is not None}
    with pytest.raises(ConfigError) as e:
        parse_config(cfg)
    assert needle in str(e.value)


def test_unknown_architecture_lists_known_ones():
    with pytest.raises(ConfigError) as e:
        resolve("Nope")
    assert "LlamaForCausalLM" in str(e.value)
    assert "LlamaForCausalLM" in known_architectures()


def test_registering_another_architecture():
    register_architecture("ToyForCausalLM", lambda cfg, gen=None, architecture="": ("toy", cfg["n"]),
                          lambda cfg: None, replace=True)
    assert parse_config({"architectures": ["ToyForCausalLM"], "n": 3}) == ("toy", 3)
    with pytest.raises(ValueError):
        register_architecture("ToyForCausalLM", None, None)


def test_missing_config_file(tmp_path):
    with pytest.raises(ConfigError):
        load_config(str(tmp_path))


def test_engine_max_context_lowers_the_position_limit_only():
    from llmengine import Engine
    assert Engine.from_random(TINY_A, 0, "fp32").max_pos == TINY_A["max_position_embeddings"]
    assert Engine.from_random(TINY_A, 0, "fp32", max_context=40).max_pos == 40
    assert Engine.from_random(TINY_A, 0, "fp32", max_context=10 ** 6).max_pos == TINY_A["max_position_embeddings"]
    with pytest.raises(ValueError):
        Engine.from_random(TINY_A, 0, "fp32", max_context=0)
    with pytest.raises(RuntimeError, match="max_pos"):
        Engine.from_random(TINY_A, 0, "fp32", max_context=8).generate([1, 2, 3, 4, 5], 8)
