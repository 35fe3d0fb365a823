"""What an execution site asks of the cache manager.

The manager has two ways of keeping things: *pages* that grow with a request's tokens (a pool per
group of sites with equal needs, a block table per request, windows) and *slots* of fixed size per
request (two copies, swapped at commit).  A spec says which of the two a site needs, brings the
tensors (their shapes are the spec's business, the manager only counts pages and rows) and makes
the view that the mixer is handed for a step.  Another kind of cache is another spec class: a
subclass of `PagedSpec` or of `SlotSpec` with its own tensors and view.  Neither the manager nor the
step function asks what class a spec is.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional

import torch

from .views import KVView, StateView

_TORCH_DTYPES = {
    "float32": torch.float32,
    "bfloat16": torch.bfloat16,
    "int32": torch.int32,
}


class SiteCacheSpec:
    """Base of every spec.  `attach` tells the manager which of its two stores the site uses."""

    def attach(self, manager: Any, site: int) -> None:
        raise NotImplementedError

    def page_bytes(self, block_size: int, element_size: int) -> int:
        """Bytes that one page id of this site costs (0 for what does not live in pages)."""
        return 0


class PagedSpec(SiteCacheSpec):
    """Something per token, kept in pages.  Equal specs (==, hash) share one pool and one free list.

    window: None keeps every token; an integer W keeps only what a query may still see, the W most
    recent positions including its own, so pages that every later query has passed are given back.
    """

    window: Optional[int] = None

    def attach(self, manager: Any, site: int) -> None:
        manager.add_paged_site(site, self)

    def page_tensors(
        self, sites: int, num_blocks: int, block_size: int, dtype: torch.dtype, device: torch.device
    ) -> dict[str, torch.Tensor]:
        """The pool's tensors by name, each [sites, num_blocks, ...]: never zeroed (stale bytes must be
        unreachable, not clean)."""
        raise NotImplementedError

    def bytes_per_token(self, element_size: int) -> int:
        raise NotImplementedError

    def page_bytes(self, block_size: int, element_size: int) -> int:
        return self.bytes_per_token(element_size) * block_size

    def view(self, pages: dict[str, torch.Tensor], **step: Any) -> Any:
        """What the mixer gets: `pages` are this site's tensors ([num_blocks, ...] each); `step` holds
        block_table, slot_mapping, block_size, writable, site, owner, tracker."""
        raise NotImplementedError


class SlotSpec(SiteCacheSpec):
    """State of fixed size per request."""

    def attach(self, manager: Any, site: int) -> None:
        manager.add_slot_site(site, self)

    def bank(self, rows: int, device: torch.device) -> torch.Tensor:
        """[rows, ...], zeroed: two rows per request slot and two spare ones."""
        raise NotImplementedError

    def view(self, tensor: torch.Tensor, read_rows: torch.Tensor, write_rows: torch.Tensor) -> Any:
        raise NotImplementedError


@dataclass(frozen=True)
class PagedKVSpec(PagedSpec):
    """Keys and values that grow with the tokens, kept in pages.

    value_head_dim: width of a value when it differs from a key's `head_dim`; 0 keeps no
    values at all (a mixer that caches one compressed vector per token and calls it the key).

    Page layout: keys [site, page, kv_head, offset in page, head_dim], the reference's inner order
    (src/mini_llm_runtime/paged_kv_cache.py:287-318); values are kept transposed inside a page,
    [site, page, kv_head, head_dim, offset in page], because the matrix cores want the index that is
    summed over (the key position, for the probability-times-value product) to be the fastest one
    of both operands.  A mixer whose kernels want another order subclasses this and overrides
    `key_page_shape` / `value_page_shape`.
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

    def key_page_shape(self, block_size: int) -> tuple[int, ...]:
        return (self.num_kv_heads, block_size, self.head_dim)

    def value_page_shape(self, block_size: int) -> tuple[int, ...]:
        return (self.num_kv_heads, self.value_dim, block_size)

    def page_tensors(self, sites, num_blocks, block_size, dtype, device):
        return {
            "key": torch.empty((sites, num_blocks, *self.key_page_shape(block_size)), dtype=dtype, device=device),
            "value": torch.empty((sites, num_blocks, *self.value_page_shape(block_size)), dtype=dtype, device=device),
        }

    def view(self, pages, **step):
        return KVView(key=pages["key"], value=pages["value"], window=self.window, **step)


@dataclass(frozen=True)
class SlotStateSpec(SlotSpec):
    """State of fixed size per request (shape per request, element type by name)."""

    shape: tuple[int, ...]
    dtype: str = "float32"

    def __post_init__(self) -> None:
        if not self.shape or any(s <= 0 for s in self.shape):
            raise ValueError("SlotStateSpec.shape must hold positive sizes")
        if self.dtype not in _TORCH_DTYPES:
            raise ValueError(f"SlotStateSpec.dtype must be one of {', '.join(_TORCH_DTYPES)}")

    def bank(self, rows, device):
        return torch.zeros((rows, *self.shape), dtype=_TORCH_DTYPES[self.dtype], device=device)

    def view(self, tensor, read_rows, write_rows):
        return StateView(tensor, read_rows, write_rows)
