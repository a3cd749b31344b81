"""Qwen2 dense decoder as a `ModelSpec` (layer order and tensor names of qwen-infer/src/model.rs:712-769)."""
from __future__ import annotations

from ..config.qwen2 import Qwen2Config
from ..config.registry import register_architecture
from ..parts.spec import (FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec,
                          ScheduleEntry)


def qwen2_spec(cfg: Qwen2Config) -> ModelSpec:
    d = cfg.derived_head_dim
    position = PositionSpec("rope_half_split", head_dim=d, theta=cfg.rope_theta,
                            max_positions=cfg.max_position_embeddings)
    layers = []
    for index in range(cfg.num_hidden_layers):
        prefix = f"model.layers.{index}"
        norm = NormSpec("rmsnorm", cfg.hidden_size, cfg.rms_norm_eps)
        layers.append(LayerSpec(
            block="pre_norm",
            mixer=MixerSpec("gqa_attention", hidden_size=cfg.hidden_size, n_heads=cfg.num_attention_heads,
                            n_kv_heads=cfg.num_key_value_heads, head_dim=d, qkv_bias=True, out_bias=False,
                            window=cfg.window_for_layer(index), position=position),
            feed_forward=FeedForwardSpec("gated_dense", hidden_size=cfg.hidden_size,
                                         intermediate_size=cfg.intermediate_size, activation=cfg.hidden_act),
            mixer_norm=norm, feed_forward_norm=norm,
            mixer_prefix=f"{prefix}.self_attn", feed_forward_prefix=f"{prefix}.mlp",
            mixer_norm_prefix=f"{prefix}.input_layernorm",
            feed_forward_norm_prefix=f"{prefix}.post_attention_layernorm"))
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
        max_positions=cfg.max_position_embeddings, embedding_name="model.embed_tokens.weight",
        layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(cfg.num_hidden_layers)),
        final_norm=NormSpec("rmsnorm", cfg.hidden_size, cfg.rms_norm_eps), final_norm_prefix="model.norm",
        tied_head=cfg.tie_word_embeddings, head_name="lm_head.weight")


register_architecture("Qwen2ForCausalLM", Qwen2Config, qwen2_spec)
