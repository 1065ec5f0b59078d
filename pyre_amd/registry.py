"""One registry from an architecture's name to its configuration class and model builder.

``config.json`` names the architecture in ``architectures[0]``; everything in the
framework (loader, engine, replay tool, command line) finds the model through
this table and nowhere else. The reference accepts any name containing "Qwen2"
(`pyre/config.py:38-43`); here the key must match exactly.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable

from pyre_amd.config.model import ConfigError, ModelConfig


@dataclass(frozen=True)
class Architecture:
    name: str
    config_cls: type[ModelConfig]
    #: ``build(config) -> pyre_amd.parts.model.ModelSpec``: the description of the
    #: layers, their order and their parts, from which the model is assembled.
    build: Callable[[Any], Any]


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(name: str, config_cls: type[ModelConfig], build: Callable) -> None:
    _ARCHITECTURES[name] = Architecture(name, config_cls, build)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def known_architectures() -> list[str]:
    _load_builtin()
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> Architecture:
    _load_builtin()
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(
            f"unknown architecture {name!r}; known: {', '.join(sorted(_ARCHITECTURES))}"
        ) from None


def architecture_of(raw: dict[str, Any]) -> Architecture:
    archs = raw.get("architectures")
    if not archs or not isinstance(archs, (list, tuple)):
        raise ConfigError("config.json has no 'architectures' list")
    return get_architecture(archs[0])


def load_config(folder_or_file: str | Path) -> ModelConfig:
    """Read ``config.json`` and return the typed configuration of its architecture."""
    p = Path(folder_or_file)
    if p.is_dir():
        p = p / "config.json"
    if not p.is_file():
        raise FileNotFoundError(f"no config.json at {p}")
    raw = json.loads(p.read_text())
    return architecture_of(raw).config_cls.from_dict(raw)


def config_from_dict(raw: dict[str, Any]) -> ModelConfig:
    return architecture_of(raw).config_cls.from_dict(raw)


_builtin_loaded = False


def _load_builtin() -> None:
    global _builtin_loaded
    if not _builtin_loaded:
        _builtin_loaded = True
        import pyre_amd.models  # noqa: F401  (registers the built-in architectures)
