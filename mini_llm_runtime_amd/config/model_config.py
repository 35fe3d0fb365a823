"""Typed model configurations read from an architecture's own config.json keys.

`ModelConfig` is the base every architecture's configuration derives from.  A
configuration holds sizes and constants only; it knows nothing about kernels or
the cache.  The builder registered beside it (see `registry.py`) turns it into a
`ModelSpec`: a per-layer list of parts with their parameters.
"""

from __future__ import annotations

import json
from dataclasses import asdict, dataclass, fields
from pathlib import Path
from typing import Any, ClassVar, Mapping


class ConfigError(ValueError):
    """A config.json that is missing keys, has bad values or names an unsupported variant."""


@dataclass(frozen=True)
class ModelConfig:
    """Base of all typed configurations; subclasses are frozen dataclasses.

    `architecture` is the registry key (config.json `architectures[0]`).
    """

    architecture: ClassVar[str] = ""
    model_type: ClassVar[str] = ""

    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> dict[str, Any]:
        """The config.json content that `from_dict` reads back to an equal object."""
        out = {f.name: getattr(self, f.name) for f in fields(self)}
        out["architectures"] = [self.architecture]
        out["model_type"] = self.model_type
        return out

    def save(self, folder: str | Path) -> Path:
        path = Path(folder) / "config.json"
        path.write_text(json.dumps(self.to_dict(), indent=2) + "\n", encoding="utf-8")
        return path


def read_config_json(model_dir: str | Path) -> dict[str, Any]:
    """Read `<model_dir>/config.json`; it must hold one JSON object.

    Reference: src/mini_llm_runtime/qwen_loader.py:16-27.
    """
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"no config.json in {model_dir}")
    data = json.loads(path.read_text(encoding="utf-8"))
    if not isinstance(data, dict):
        raise ConfigError(f"{path} must hold a JSON object, found {type(data).__name__}")
    return data


def require_keys(data: Mapping[str, Any], keys: tuple[str, ...], where: str) -> None:
    missing = [k for k in keys if k not in data]
    if missing:
        raise ConfigError(f"{where}: config.json lacks the keys {', '.join(missing)}")


def positive_int(data: Mapping[str, Any], key: str) -> int:
    value = data[key]
    if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
        raise ConfigError(f"config key {key!r} must be a positive integer, found {value!r}")
    return int(value)


def positive_float(data: Mapping[str, Any], key: str) -> float:
    value = data[key]
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not value > 0:
        raise ConfigError(f"config key {key!r} must be a positive number, found {value!r}")
    return float(value)


__all__ = [
    "ConfigError",
    "ModelConfig",
    "asdict",
    "positive_float",
    "positive_int",
    "read_config_json",
    "require_keys",
]
