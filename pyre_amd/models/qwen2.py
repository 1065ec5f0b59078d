"""Qwen2 / Qwen2.5 dense decoder as a list of parts (`pyre/model.py:142-175`).

Every layer is the same pre-norm block: RMSNorm, grouped-query attention with bias
on q/k/v and none on the output projection, half-split rotary positions over the
whole head, RMSNorm, SwiGLU. Tensor names are the checkpoint's
(`pyre/model.py:1-5,156-158`).
"""

from __future__ import annotations

from pyre_amd.config.model import Qwen2Config
from pyre_amd.parts.base import (AttentionSpec, BlockSpec, EmbeddingSpec, LayerCall, LMHeadSpec,
                                 ModelSpec, RMSNormSpec, RotarySpec, SwiGLUSpec)
from pyre_amd.registry import register_architecture


def build_qwen2(cfg: Qwen2Config) -> ModelSpec:
    rotary = RotarySpec(cfg.head_dim, cfg.rope_theta, cfg.max_position_embeddings)
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}"
        layers.append(BlockSpec(
            mixer=AttentionSpec(cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads,
                                cfg.head_dim, rotary, f"{p}.self_attn", qkv_bias=True, out_bias=False),
            mixer_norm=RMSNormSpec(cfg.hidden_size, cfg.rms_norm_eps, f"{p}.input_layernorm"),
            feed_forward=SwiGLUSpec(cfg.hidden_size, cfg.intermediate_size, f"{p}.mlp"),
            feed_forward_norm=RMSNormSpec(cfg.hidden_size, cfg.rms_norm_eps, f"{p}.post_attention_layernorm"),
        ))
    embedding = EmbeddingSpec(cfg.vocab_size, cfg.hidden_size)
    return ModelSpec(
        hidden_size=cfg.hidden_size, vocab_size=cfg.vocab_size,
        max_positions=cfg.max_position_embeddings, embedding=embedding, layers=tuple(layers),
        schedule=tuple(LayerCall(i) for i in range(cfg.num_hidden_layers)),
        final_norm=RMSNormSpec(cfg.hidden_size, cfg.rms_norm_eps, "model.norm"),
        head=LMHeadSpec(cfg.vocab_size, cfg.hidden_size,
                        tied_to=embedding.name if cfg.tie_word_embeddings else None),
    )


register_architecture(Qwen2Config.architecture, Qwen2Config, build_qwen2)
