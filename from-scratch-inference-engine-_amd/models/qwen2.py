"""Qwen2 dense decoder: which parts, in which order, from which checkpoint tensors."""

from __future__ import annotations

from typing import List

from ..config.qwen2 import Qwen2Config
from ..parts.base import make_part
from ..parts.embedding import LMHead, TokenEmbedding
from ..weights.loader import ParamBinding, TensorSpec
from .registry import register_architecture
from .spec import LayerCall, ModelSpec, bind


def build_qwen2(cfg: Qwen2Config) -> ModelSpec:
    """Every layer: RMSNorm -> GQA attention (q/k/v bias, RoPE, no o bias) -> residual ->
    RMSNorm -> SwiGLU -> residual; then the final RMSNorm and the LM head (tied to the embedding
    table or a tensor of its own).  Tensor names are those the reference reads
    (src/cuda/model.cu:750-766)."""
    h, nh, nkv, hd, inter = (cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads,
                             cfg.head_dim, cfg.intermediate_size)
    q_dim, kv_dim = nh * hd, nkv * hd
    bindings: List[ParamBinding] = []

    embedding = TokenEmbedding(cfg.vocab_size, h)
    embed_spec = TensorSpec("model.embed_tokens.weight", (cfg.vocab_size, h))
    bind(bindings, embedding, "weight", [embed_spec])

    layers = []
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        position = make_part("position", "rope", head_dim=hd, theta=cfg.rope_theta)
        mixer = make_part("mixer", "gqa_attention", hidden_size=h, n_heads=nh, n_kv_heads=nkv, head_dim=hd,
                          qkv_bias=cfg.attention_qkv_bias, position=position, window=None)
        ffn = make_part("feed_forward", "swiglu", hidden_size=h, intermediate_size=inter)
        norm1 = make_part("norm", "rms_norm", hidden_size=h, eps=cfg.rms_norm_eps)
        norm2 = make_part("norm", "rms_norm", hidden_size=h, eps=cfg.rms_norm_eps)
        layers.append(make_part("block", "pre_norm", mixer_norm=norm1, mixer=mixer, ffn_norm=norm2, ffn=ffn))

        bind(bindings, norm1, "weight", [TensorSpec(p + "input_layernorm.weight", (h,), "norm")])
        bind(bindings, norm2, "weight", [TensorSpec(p + "post_attention_layernorm.weight", (h,), "norm")])
        bind(bindings, mixer, "qkv_weight", [TensorSpec(p + "self_attn.q_proj.weight", (q_dim, h)),
                                             TensorSpec(p + "self_attn.k_proj.weight", (kv_dim, h)),
                                             TensorSpec(p + "self_attn.v_proj.weight", (kv_dim, h))])
        if cfg.attention_qkv_bias:
            bind(bindings, mixer, "qkv_bias", [TensorSpec(p + "self_attn.q_proj.bias", (q_dim,), "bias"),
                                               TensorSpec(p + "self_attn.k_proj.bias", (kv_dim,), "bias"),
                                               TensorSpec(p + "self_attn.v_proj.bias", (kv_dim,), "bias")])
        bind(bindings, mixer, "o_weight", [TensorSpec(p + "self_attn.o_proj.weight", (h, q_dim))])
        bind(bindings, ffn, "gate_up_weight", [TensorSpec(p + "mlp.gate_proj.weight", (inter, h)),
                                               TensorSpec(p + "mlp.up_proj.weight", (inter, h))])
        bind(bindings, ffn, "down_weight", [TensorSpec(p + "mlp.down_proj.weight", (h, inter))])

    final_norm = make_part("norm", "rms_norm", hidden_size=h, eps=cfg.rms_norm_eps)
    bind(bindings, final_norm, "weight", [TensorSpec("model.norm.weight", (h,), "norm")])

    lm_head = LMHead(h, cfg.vocab_size)
    if cfg.tie_word_embeddings:
        bind(bindings, lm_head, "weight", [embed_spec])
    else:
        bind(bindings, lm_head, "weight", [TensorSpec("lm_head.weight", (cfg.vocab_size, h))])

    return ModelSpec(
        config=cfg, embedding=embedding, layers=layers,
        schedule=[LayerCall(l) for l in range(cfg.num_hidden_layers)],
        final_norm=final_norm, lm_head=lm_head, bindings=bindings,
        # a tied checkpoint may still carry a copy of the head: it is not read
        ignore_unexpected=("lm_head.weight",) if cfg.tie_word_embeddings else (),
    )


register_architecture("Qwen2ForCausalLM", Qwen2Config, build_qwen2)
