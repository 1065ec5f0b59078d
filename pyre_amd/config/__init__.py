from pyre_amd.config.engine import EngineConfig
from pyre_amd.config.model import ConfigError, ModelConfig, Qwen2Config
from pyre_amd.config.presets import PRESETS, preset

__all__ = ["ConfigError", "EngineConfig", "ModelConfig", "Qwen2Config", "PRESETS", "preset"]
