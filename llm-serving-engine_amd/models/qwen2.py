"""Qwen2 / Qwen2.5 dense decoder as a list of parts (reference `model.py:191-258`)."""

from __future__ import annotations

import math

from ..config.model import Qwen2Config
from ..parts import (
    AttentionSpec,
    GatedMLPSpec,
    LayerDefinition,
    LayerRun,
    ModelSpec,
    PreNormBlockSpec,
    RMSNormSpec,
    RotarySpec,
)
from ..registry import register_architecture


def qwen2_spec(config: Qwen2Config) -> ModelSpec:
    norm = RMSNormSpec(config.hidden_size, config.rms_norm_eps)
    rotary = RotarySpec(config.head_dim, config.rope_theta, config.rope_pairing)
    feed_forward = GatedMLPSpec(config.hidden_size, config.intermediate_size, "silu")
    layers = []
    for index in range(config.num_layers):
        attention = AttentionSpec(
            hidden_size=config.hidden_size,
            num_heads=config.num_attention_heads,
            num_kv_heads=config.num_key_value_heads,
            head_dim=config.head_dim,
            scale=1.0 / math.sqrt(config.head_dim),  # `model.py:133,144`
            position=rotary,
            qkv_bias=config.attention_bias,
            out_bias=False,  # `model.py:66`
            window=config.layer_window(index),
        )
        block = PreNormBlockSpec(norm, attention, norm, feed_forward)
        layers.append(LayerDefinition(f"model.layers.{index}.", block))
    return ModelSpec(
        vocab_size=config.vocab_size,
        hidden_size=config.hidden_size,
        layers=tuple(layers),
        run_order=tuple(LayerRun(index) for index in range(config.num_layers)),
        final_norm=norm,
        tie_embeddings=config.tie_word_embeddings,
    )


register_architecture("Qwen2ForCausalLM", Qwen2Config, qwen2_spec, model_types=("qwen2",))
