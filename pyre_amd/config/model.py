"""Typed model configurations, read from an architecture's own ``config.json`` keys.

Every size and constant of a model comes from here; no part of the engine holds
a literal size. The keys read for Qwen2 are the ones the reference reads
(`pyre/config.py:34-62`), with the same defaults, plus three keys the reference
silently ignores and this engine insists on seeing in a supported state
(``use_sliding_window``, ``hidden_act``, ``rope_scaling``).
"""

from __future__ import annotations

import json
from dataclasses import asdict, dataclass, fields
from pathlib import Path
from typing import Any, ClassVar


class ConfigError(ValueError):
    """A config.json that is incomplete, inconsistent or asks for something unsupported."""


@dataclass(frozen=True)
class ModelConfig:
    """Base of all architecture configurations.

    A subclass names its architecture (the string in ``architectures[0]``), lists
    its fields, and implements :meth:`from_dict` and :meth:`to_dict` so that a
    configuration written by :meth:`to_dict` is read back unchanged.
    """

    architecture: ClassVar[str] = ""

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> dict[str, Any]:
        raise NotImplementedError

    @classmethod
    def from_json(cls, path: str | Path) -> "ModelConfig":
        return cls.from_dict(json.loads(Path(path).read_text()))

    def save(self, folder: str | Path) -> None:
        Path(folder).mkdir(parents=True, exist_ok=True)
        (Path(folder) / "config.json").write_text(json.dumps(self.to_dict(), indent=2) + "\n")


def _require(raw: dict[str, Any], key: str, kind=int):
    if key not in raw:
        raise ConfigError(f"config.json has no {key!r}")
    value = raw[key]
    if kind is int and (isinstance(value, bool) or not isinstance(value, int)):
        raise ConfigError(f"config.json: {key!r} must be an integer, got {value!r}")
    return value


@dataclass(frozen=True)
class Qwen2Config(ModelConfig):
    """Qwen2 / Qwen2.5 dense decoder (`pyre/config.py:15-27`)."""

    architecture: ClassVar[str] = "Qwen2ForCausalLM"

    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    vocab_size: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    max_position_embeddings: int
    head_dim: int

    @property
    def n_rep(self) -> int:
        """Query heads per key/value head (`pyre/config.py:29-32`)."""
        return self.num_attention_heads // self.num_key_value_heads

    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    def __post_init__(self) -> None:
        for f in fields(self):
            v = getattr(self, f.name)
            if f.type == "int" and (not isinstance(v, int) or isinstance(v, bool) or v <= 0):
                raise ConfigError(f"{f.name} must be a positive integer, got {v!r}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads ({self.num_attention_heads}) is not a multiple of "
                f"num_key_value_heads ({self.num_key_value_heads})"
            )
        if self.head_dim % 2:
            raise ConfigError(f"head_dim must be even for rotary pairs, got {self.head_dim}")
        if not (self.rms_norm_eps > 0):
            raise ConfigError(f"rms_norm_eps must be positive, got {self.rms_norm_eps!r}")
        if not (self.rope_theta > 0):
            raise ConfigError(f"rope_theta must be positive, got {self.rope_theta!r}")

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "Qwen2Config":
        hidden = _require(raw, "hidden_size")
        n_heads = _require(raw, "num_attention_heads")
        # The reference admits every config silently; what it cannot compute
        # (`pyre/model.py:111-120` is pure causal, `:139` is SiLU, `:41-51` has no
        # frequency scaling) is refused here instead of being computed wrongly.
        if raw.get("use_sliding_window", False):
            raise ConfigError("use_sliding_window=true is not supported for Qwen2ForCausalLM")
        if raw.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"hidden_act must be 'silu', got {raw['hidden_act']!r}")
        if raw.get("rope_scaling") is not None:
            raise ConfigError("rope_scaling is not supported for Qwen2ForCausalLM")
        # `pyre/config.py:47-48`: head_dim defaults to hidden_size // heads.
        head_dim = raw.get("head_dim") or hidden // n_heads
        return cls(
            hidden_size=hidden,
            intermediate_size=_require(raw, "intermediate_size"),
            num_hidden_layers=_require(raw, "num_hidden_layers"),
            num_attention_heads=n_heads,
            num_key_value_heads=raw.get("num_key_value_heads", n_heads),
            vocab_size=_require(raw, "vocab_size"),
            rms_norm_eps=float(raw.get("rms_norm_eps", 1e-6)),
            rope_theta=float(raw.get("rope_theta", 10000.0)),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            max_position_embeddings=raw.get("max_position_embeddings", 32768),
            head_dim=head_dim,
        )

    def to_dict(self) -> dict[str, Any]:
        out = {"architectures": [self.architecture], "model_type": "qwen2"}
        out.update(asdict(self))
        out.update(hidden_act="silu", use_sliding_window=False, rope_scaling=None)
        return out
