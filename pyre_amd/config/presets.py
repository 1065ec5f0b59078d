"""Named model shapes: two tiny test shapes and the published Qwen2.5 sizes.

A preset is only a ``config.json`` dictionary; it goes through the same
``from_dict`` as a file does.
"""

from __future__ import annotations

from typing import Any

from pyre_amd.config.model import Qwen2Config


def _qwen2(**kw: Any) -> dict[str, Any]:
    base = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
            "use_sliding_window": False}
    base.update(kw)
    return base


PRESETS: dict[str, dict[str, Any]] = {
    "tiny-a": _qwen2(
        num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2,
        head_dim=16, intermediate_size=176, vocab_size=512, rope_theta=1e4, rms_norm_eps=1e-6,
        tie_word_embeddings=True, max_position_embeddings=256),
    "tiny-b": _qwen2(
        num_hidden_layers=3, hidden_size=96, num_attention_heads=8, num_key_value_heads=2,
        head_dim=12, intermediate_size=256, vocab_size=1000, rope_theta=1e6, rms_norm_eps=1e-5,
        tie_word_embeddings=False, max_position_embeddings=512),
    "qwen2.5-1.5b": _qwen2(
        num_hidden_layers=28, hidden_size=1536, num_attention_heads=12, num_key_value_heads=2,
        head_dim=128, intermediate_size=8960, vocab_size=151936, rope_theta=1e6,
        rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=32768),
    "qwen2.5-7b": _qwen2(
        num_hidden_layers=28, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4,
        head_dim=128, intermediate_size=18944, vocab_size=152064, rope_theta=1e6,
        rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=32768),
    "qwen2.5-32b": _qwen2(
        num_hidden_layers=64, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
        head_dim=128, intermediate_size=27648, vocab_size=152064, rope_theta=1e6,
        rms_norm_eps=1e-5, tie_word_embeddings=False, max_position_embeddings=32768),
}


def preset(name: str, **overrides: Any) -> Qwen2Config:
    if name not in PRESETS:
        raise KeyError(f"unknown preset {name!r}; known: {', '.join(sorted(PRESETS))}")
    raw = dict(PRESETS[name])
    raw.update(overrides)
    from pyre_amd.registry import config_from_dict

    return config_from_dict(raw)
