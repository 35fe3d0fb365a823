"""Architectures: each module registers one name with its configuration and builder."""

from . import qwen2  # noqa: F401  (registers Qwen2ForCausalLM)
from .registry import (
    ARCHITECTURES,
    Architecture,
    architecture_of,
    build_model,
    build_spec,
    config_from_dict,
    load_config,
    register_architecture,
    unregister_architecture,
)

__all__ = [
    "ARCHITECTURES",
    "Architecture",
    "architecture_of",
    "build_model",
    "build_spec",
    "config_from_dict",
    "load_config",
    "register_architecture",
    "unregister_architecture",
]
