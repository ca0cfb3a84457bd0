"""Typed configuration and the architecture registry."""

import json

import pytest

import helpers
from from_scratch_inference_engine_amd.config import ConfigError, Qwen2Config
from from_scratch_inference_engine_amd.models import (build_model_spec, known_architectures, load_config,
                                                      parse_config, register_architecture)


def test_defaults_follow_the_reference():
    # tests/cpp/test_safetensors.cpp:105-119: 896 / 14 -> head_dim 64; qwen2 -> q/k/v bias
    c = parse_config({"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_size": 896,
                      "num_hidden_layers": 24, "num_attention_heads": 14, "num_key_value_heads": 2,
                      "intermediate_size": 4864, "vocab_size": 151936})
    assert isinstance(c, Qwen2Config)
    assert (c.head_dim, c.attention_qkv_bias, c.rope_theta, c.rms_norm_eps) == (64, True, 10000.0, 1e-6)
    assert c.tie_word_embeddings is False and c.max_position_embeddings == 0 and c.eos_token_id == -1
    # kv heads default to the heads
    c = parse_config({"architectures": ["Qwen2ForCausalLM"], "hidden_size": 64, "num_hidden_layers": 1,
                      "num_attention_heads": 4, "intermediate_size": 8, "vocab_size": 10})
    assert c.num_key_value_heads == 4 and c.attention_qkv_bias is False  # not qwen2: attention_bias, default off
    # explicit head_dim and attention_bias (test_safetensors.cpp:121-140)
    c = parse_config({"architectures": ["Qwen2ForCausalLM"], "model_type": "llama", "hidden_size": 64,
                      "num_hidden_layers": 1, "num_attention_heads": 4, "head_dim": 32, "attention_bias": True,
                      "intermediate_size": 8, "vocab_size": 10, "eos_token_id": [5, 6]})
    assert c.head_dim == 32 and c.attention_qkv_bias is True and c.eos_token_id == 5


def test_every_size_comes_from_config():
    a, b = parse_config(helpers.TINY_A), parse_config(helpers.TINY_B)
    assert (a.hidden_size, a.num_hidden_layers, a.num_attention_heads, a.num_key_value_heads, a.head_dim,
            a.intermediate_size, a.vocab_size, a.rope_theta, a.rms_norm_eps, a.tie_word_embeddings,
            a.max_position_embeddings) == (64, 2, 4, 2, 16, 176, 256, 1e4, 1e-6, True, 128)
    assert (b.hidden_size, b.num_hidden_layers, b.num_attention_heads, b.num_key_value_heads, b.head_dim,
            b.intermediate_size, b.vocab_size, b.rope_theta, b.rms_norm_eps, b.tie_word_embeddings,
            b.max_position_embeddings, b.eos_token_id) == (192, 3, 6, 1, 32, 320, 509, 1e6, 1e-5, False, 256, 7)
    # and reaches the parts
    spec = build_model_spec(b)
    blk = spec.layers[2]
    assert (blk.mixer.n_heads, blk.mixer.n_kv, blk.mixer.head_dim, blk.mixer.position.theta) == (6, 1, 32, 1e6)
    assert blk.mixer_norm.eps == 1e-5 and blk.ffn.intermediate_size == 320 and len(spec.layers) == 3
    assert Qwen2Config.from_dict(b.to_dict()) == b


@pytest.mark.parametrize("patch, message", [
    ({"num_attention_heads": 0}, "num_attention_heads"),
    ({"hidden_size": None}, "hidden_size"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"type": "yarn", "factor": 4.0}}, "rope_scaling"),
    ({"use_sliding_window": True}, "sliding"),
    ({"head_dim": 15}, "even"),
    ({"vocab_size": "many"}, "vocab_size"),
])
def test_refused_values(patch, message):
    raw = dict(helpers.TINY_A)
    raw.update(patch)
    if patch.get("hidden_size", 0) is None:
        del raw["hidden_size"]
    with pytest.raises(ConfigError, match=message):
        parse_config(raw)


def test_registry(tmp_path):
    assert "Qwen2ForCausalLM" in known_architectures()
    with pytest.raises(ConfigError, match="not registered.*Qwen2ForCausalLM"):
        parse_config({"architectures": ["NoSuchModel"]})
    with pytest.raises(ConfigError, match="architectures"):
        parse_config({"hidden_size": 8})
    (tmp_path / "config.json").write_text(json.dumps(helpers.TINY_A))
    assert load_config(tmp_path).hidden_size == 64
    with pytest.raises(ConfigError, match="no config.json"):
        load_config(tmp_path / "nowhere")
    (tmp_path / "config.json").write_text("{broken")
    with pytest.raises(ConfigError, match="invalid JSON"):
        load_config(tmp_path)
    # another architecture registers without touching the engine's files
    register_architecture("ToyForTest", Qwen2Config, lambda cfg: "spec")
    raw = dict(helpers.TINY_A, architectures=["ToyForTest"])
    assert build_model_spec(parse_config(raw)) == "spec"
