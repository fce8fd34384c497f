"""Qwen2: from its configuration to a plan of parts.

The architecture is pre-norm blocks of grouped-query attention (q/k/v bias, no o bias,
half-split rotary encoding) and a SwiGLU feed-forward, RMSNorm everywhere, a tied or untied
head (src/turboserve/engine/model/model.py:51-108, layers.py:311-487).  With
``use_sliding_window`` the layers from ``max_window_layers`` on see a window of keys.
"""

from __future__ import annotations

from turboserve_amd.config.model_config import Qwen2Config
from turboserve_amd.models.decoder import LayerCall, LayerSpec, ModelPlan
from turboserve_amd.parts.base import PartSpec
from turboserve_amd.parts.ends import standard_ends


def qwen2_plan(config: Qwen2Config) -> ModelPlan:
    norm = PartSpec("rmsnorm", {"size": config.hidden_size, "eps": config.rms_norm_eps})
    position = PartSpec(
        "rope",
        {
            "head_dim": config.head_dim,
            "theta": config.rope_theta,
            "scaling_factor": config.rope_scaling_factor,
            "max_positions": config.max_position_embeddings,
        },
    )
    feed_forward = PartSpec(
        "swiglu", {"hidden_size": config.hidden_size, "intermediate_size": config.intermediate_size}
    )
    layers = []
    for index in range(config.num_hidden_layers):
        mixer = PartSpec(
            "gqa_attention",
            {
                "hidden_size": config.hidden_size,
                "num_heads": config.num_attention_heads,
                "num_kv_heads": config.num_key_value_heads,
                "head_dim": config.head_dim,
                "scale": config.attn_scale,
                "qkv_bias": config.qkv_bias,
                "out_bias": config.o_proj_bias,
                "window": config.layer_window(index),
                "position": position,
            },
        )
        block = PartSpec(
            "prenorm",
            {"mixer": mixer, "feed_forward": feed_forward, "mixer_norm": norm, "ff_norm": norm},
        )
        layers.append(LayerSpec(prefix=f"model.layers.{index}", block=block))
    return ModelPlan(
        vocab_size=config.vocab_size,
        hidden_size=config.hidden_size,
        layers=tuple(layers),
        schedule=tuple(LayerCall(i) for i in range(config.num_hidden_layers)),
        **standard_ends(config.vocab_size, config.hidden_size, norm, tie_head=config.tie_word_embeddings),
    )
