"""Configuration: typed model configs, the architecture registry, engine options."""

from .engine_config import POLICIES, EngineConfig, blocks_for_capacity
from .model_config import ConfigError, Qwen2Config, read_config_json
from .registry import build_model, known_architectures, register_architecture, resolve

__all__ = [
    "ConfigError", "EngineConfig", "POLICIES", "Qwen2Config", "blocks_for_capacity",
    "build_model", "known_architectures", "read_config_json", "register_architecture", "resolve",
]
