"""Typed configurations."""

from .model_config import ConfigError, ModelConfig, read_config_json
from .bubitar import BubitarConfig
from .fedolorn import FedolornConfig
from .qwen2 import Qwen2Config

__all__ = ["BubitarConfig", "ConfigError", "FedolornConfig", "ModelConfig", "Qwen2Config", "read_config_json"]
