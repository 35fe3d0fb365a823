"""Named config.json files for the random-weights mode (benchmark shapes and tiny models)."""

from __future__ import annotations

import json
from pathlib import Path
from typing import Any

_FOLDER = Path(__file__).resolve().parent / "presets"


def preset_names() -> tuple[str, ...]:
    return tuple(sorted(p.stem for p in _FOLDER.glob("*.json")))


def load_preset(name: str) -> dict[str, Any]:
    """The config.json content of a preset name, or of a path to a JSON file."""
    path = _FOLDER / f"{name}.json"
    if not path.is_file():
        path = Path(name)
    if not path.is_file():
        raise FileNotFoundError(f"no preset or file {name!r}; presets: {', '.join(preset_names())}")
    return json.loads(path.read_text(encoding="utf-8"))
