"""Configuration of the Qwen2 dense decoder (architecture name ``Qwen2ForCausalLM``)."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .base import ConfigError, ModelConfig, checked_float, checked_int, end_token_of, required_int


@dataclass(frozen=True)
class Qwen2Config(ModelConfig):
    """Keys and defaults follow the reference's parser (src/model/model_config.cpp:9-33):
    ``num_key_value_heads`` defaults to ``num_attention_heads``, ``head_dim`` to
    ``hidden_size / num_attention_heads``, ``rope_theta`` to 10000, ``rms_norm_eps`` to 1e-6,
    ``tie_word_embeddings`` to false, ``max_position_embeddings`` to 0 (no limit);
    ``model_type == "qwen2"`` switches the q/k/v bias on, any other model type follows
    ``attention_bias``.  Beyond the reference, values the engine cannot run are refused here
    instead of being ignored: another activation than SiLU, RoPE scaling, a sliding window.
    """

    hidden_size: int = 0
    num_hidden_layers: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    intermediate_size: int = 0
    vocab_size: int = 0
    max_position_embeddings: int = 0
    rope_theta: float = 10000.0
    rms_norm_eps: float = 1e-6
    tie_word_embeddings: bool = False
    attention_qkv_bias: bool = True
    hidden_act: str = "silu"
    model_type: str = "qwen2"
    eos_token_id: int = -1

    @property
    def max_positions(self) -> int:
        return self.max_position_embeddings

    @property
    def end_token(self) -> int:
        return self.eos_token_id

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "Qwen2Config":
        archs = raw.get("architectures") or ["Qwen2ForCausalLM"]
        model_type = str(raw.get("model_type", ""))
        hidden = required_int(raw, "hidden_size")
        layers = required_int(raw, "num_hidden_layers")
        heads = required_int(raw, "num_attention_heads")
        kv_heads = checked_int(raw.get("num_key_value_heads", heads), "num_key_value_heads")
        if "head_dim" in raw and raw["head_dim"] is not None:
            head_dim = checked_int(raw["head_dim"], "head_dim")
        else:
            if hidden % heads:
                raise ConfigError(
                    f"config.json: hidden_size {hidden} is not a multiple of num_attention_heads "
                    f"{heads} and no head_dim is given")
            head_dim = hidden // heads
        if heads % kv_heads:
            raise ConfigError(
                f"config.json: num_attention_heads {heads} is not a multiple of "
                f"num_key_value_heads {kv_heads}")
        if head_dim % 2:
            raise ConfigError(f"config.json: head_dim {head_dim} must be even for rotary pairs")
        act = str(raw.get("hidden_act", "silu"))
        if act != "silu":
            raise ConfigError(f"config.json: hidden_act '{act}' is not supported (only 'silu')")
        if raw.get("rope_scaling") not in (None, {}):
            raise ConfigError("config.json: rope_scaling is not supported")
        if raw.get("use_sliding_window", False):
            raise ConfigError("config.json: use_sliding_window=true is not supported")
        qkv_bias = True if model_type == "qwen2" else bool(raw.get("attention_bias", False))
        return cls(
            architecture=str(archs[0]),
            hidden_size=hidden,
            num_hidden_layers=layers,
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=required_int(raw, "intermediate_size"),
            vocab_size=required_int(raw, "vocab_size"),
            max_position_embeddings=checked_int(raw.get("max_position_embeddings", 0),
                                                "max_position_embeddings", 0),
            rope_theta=checked_float(raw.get("rope_theta", 10000.0), "rope_theta"),
            rms_norm_eps=checked_float(raw.get("rms_norm_eps", 1e-6), "rms_norm_eps", positive=False),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            attention_qkv_bias=qkv_bias,
            hidden_act=act,
            model_type=model_type,
            eos_token_id=end_token_of(raw),
        )

    def to_dict(self) -> dict:
        return {
            "architectures": [self.architecture],
            "model_type": self.model_type,
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rope_theta": self.rope_theta,
            "rms_norm_eps": self.rms_norm_eps,
            "tie_word_embeddings": self.tie_word_embeddings,
            "attention_bias": self.attention_qkv_bias,
            "hidden_act": self.hidden_act,
            "use_sliding_window": False,
            **({"eos_token_id": self.eos_token_id} if self.eos_token_id >= 0 else {}),
        }
