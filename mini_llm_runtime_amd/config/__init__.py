"""Typed configurations."""

from .model_config import ConfigError, ModelConfig, read_config_json
from .qwen2 import Qwen2Config

__all__ = ["ConfigError", "ModelConfig", "Qwen2Config", "read_config_json"]
