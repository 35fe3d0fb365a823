"""Registries of part kinds.  A part kind is a class constructed from the keyword
arguments of its `PartSpec`; registering a new class under a new name is all it
takes to make it available to model builders (tests register toy parts this way).
"""

from __future__ import annotations

from typing import Any, Callable

from .spec import PartSpec

CATEGORIES = ("mixer", "feed_forward", "norm", "position", "block")

_REGISTRY: dict[str, dict[str, Callable[..., Any]]] = {c: {} for c in CATEGORIES}


def register_part(category: str, kind: str, factory: Callable[..., Any] | None = None, *, replace: bool = False):
    """Register `factory` (a class) as `kind` of `category`; usable as a decorator."""
    if category not in _REGISTRY:
        raise KeyError(f"unknown part category {category!r}; known: {', '.join(CATEGORIES)}")

    def _do(obj: Callable[..., Any]) -> Callable[..., Any]:
        if kind in _REGISTRY[category] and not replace and _REGISTRY[category][kind] is not obj:
            raise ValueError(f"{category} kind {kind!r} is already registered")
        _REGISTRY[category][kind] = obj
        return obj

    if factory is None:
        return _do
    return _do(factory)


def unregister_part(category: str, kind: str) -> None:
    _REGISTRY[category].pop(kind, None)


def part_kinds(category: str) -> tuple[str, ...]:
    return tuple(sorted(_REGISTRY[category]))


def build_part(category: str, spec: PartSpec, **extra: Any) -> Any:
    try:
        factory = _REGISTRY[category][spec.kind]
    except KeyError:
        raise KeyError(
            f"unknown {category} kind {spec.kind!r}; known: {', '.join(part_kinds(category)) or '(none)'}"
        ) from None
    return factory(**dict(spec.params), **extra)
