"""One registry from an architecture's name to its configuration class and its
builder.  `config.json["architectures"][0]` is the key, as everywhere in the
framework; a config without that key is looked up by its `model_type`.

The reference has no registry: its model type gate is an `if`
(src/mini_llm_runtime/qwen_config.py:61) and its runner is wired to one model.
"""

from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable, Mapping, Type

from ..config.model_config import ConfigError, ModelConfig, read_config_json
from ..parts.model import DecoderModel
from ..parts.spec import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: Type[ModelConfig]
    build_spec: Callable[[ModelConfig], ModelSpec]


ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(
    name: str,
    config_class: Type[ModelConfig],
    build_spec: Callable[[Any], ModelSpec],
    *,
    replace: bool = False,
) -> Architecture:
    if name in ARCHITECTURES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    arch = Architecture(name, config_class, build_spec)
    ARCHITECTURES[name] = arch
    return arch


def unregister_architecture(name: str) -> None:
    ARCHITECTURES.pop(name, None)


def architecture_of(data: Mapping[str, Any]) -> Architecture:
    names = data.get("architectures")
    if isinstance(names, (list, tuple)) and names:
        name = names[0]
        if name in ARCHITECTURES:
            return ARCHITECTURES[name]
        raise ConfigError(
            f"unknown architecture {name!r}; registered: {', '.join(sorted(ARCHITECTURES)) or '(none)'}"
        )
    model_type = data.get("model_type")
    for arch in ARCHITECTURES.values():
        if arch.config_class.model_type and arch.config_class.model_type == model_type:
            return arch
    raise ConfigError(
        f"config.json names no registered architecture (architectures={names!r}, model_type={model_type!r}); "
        f"registered: {', '.join(sorted(ARCHITECTURES)) or '(none)'}"
    )


def config_from_dict(data: Mapping[str, Any]) -> ModelConfig:
    return architecture_of(data).config_class.from_dict(data)


def load_config(model_dir: str | Path) -> ModelConfig:
    return config_from_dict(read_config_json(model_dir))


def build_spec(config: ModelConfig) -> ModelSpec:
    try:
        arch = ARCHITECTURES[config.architecture]
    except KeyError:
        raise ConfigError(f"architecture {config.architecture!r} is not registered") from None
    return arch.build_spec(config)


def build_model(config: ModelConfig) -> DecoderModel:
    """The model of a configuration, with unbound parameters."""
    return DecoderModel(build_spec(config))
