"""What an execution site asks of the cache manager."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass(frozen=True)
class PagedKVSpec:
    """Keys and values that grow with the tokens, kept in pages.

    window: None keeps every key; an integer W keeps only what a query may still
    see, the W most recent positions including its own, so pages that every later
    query has passed are given back.
    """

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None

    def __post_init__(self) -> None:
        if self.num_kv_heads <= 0 or self.head_dim <= 0:
            raise ValueError("PagedKVSpec sizes must be > 0")
        if self.window is not None and self.window <= 0:
            raise ValueError("PagedKVSpec.window must be > 0 or None")


@dataclass(frozen=True)
class SlotStateSpec:
    """State of fixed size per request (shape per request, element type by name)."""

    shape: tuple[int, ...]
    dtype: str = "float32"

    def __post_init__(self) -> None:
        if not self.shape or any(s <= 0 for s in self.shape):
            raise ValueError("SlotStateSpec.shape must hold positive sizes")
