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
    value_head_dim: width of a value when it differs from a key's `head_dim`; 0 keeps no
    values at all (a mixer that caches one compressed vector per token and calls it the key).
    """

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    value_head_dim: Optional[int] = None

    def __post_init__(self) -> None:
        if self.num_kv_heads <= 0 or self.head_dim <= 0:
            raise ValueError("PagedKVSpec sizes must be > 0")
        if self.window is not None and self.window <= 0:
            raise ValueError("PagedKVSpec.window must be > 0 or None")
        if self.value_head_dim is not None and self.value_head_dim < 0:
            raise ValueError("PagedKVSpec.value_head_dim must be >= 0 or None")

    @property
    def value_dim(self) -> int:
        return self.head_dim if self.value_head_dim is None else self.value_head_dim

    def bytes_per_token(self, element_size: int) -> int:
        """Keys and values of one token of one site."""
        return self.num_kv_heads * (self.head_dim + self.value_dim) * element_size


@dataclass(frozen=True)
class SlotStateSpec:
    """State of fixed size per request (shape per request, element type by name)."""

    shape: tuple[int, ...]
    dtype: str = "float32"

    def __post_init__(self) -> None:
        if not self.shape or any(s <= 0 for s in self.shape):
            raise ValueError("SlotStateSpec.shape must hold positive sizes")
