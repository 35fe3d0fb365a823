"""What a mixer is handed of its execution site's cache for one step.  A view is made by the
site's cache spec (`cache/spec.py`), so a new kind of cache brings a view of its own."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional

import torch


@dataclass
class KVView:
    """Pages of one site: keys [page, kv_head, offset, head_dim], values
    [page, kv_head, head_dim, offset], the block table rows of the step's entries
    and the slot of each new token."""

    key: torch.Tensor
    value: torch.Tensor
    block_table: torch.Tensor  # [R, max pages] int32, -1 where there is no page
    slot_mapping: torch.Tensor  # [T] int32: page * block_size + offset
    block_size: int
    window: Optional[int]
    writable: bool  # False when the site reads another site's cache
    site: int = -1  # the execution site this view was made for
    owner: int = -1  # the site that owns the pages (== site when writable)
    tracker: Any = None  # the cache manager's visibility check, when it is switched on

    def written(self) -> None:
        """The mixer reports that it has stored the step's keys and values of this site."""
        if self.tracker is not None:
            self.tracker.note_write(self.site, self.owner)

    def reading(self) -> None:
        """The mixer reports that it is about to read this site's pages, the step's own
        tokens included.  With the check switched on this raises unless the owning site
        has written them."""
        if self.tracker is not None:
            self.tracker.note_read(self.site, self.owner)


@dataclass
class StateView:
    """Fixed-size state of one site: read rows `read_rows`, write rows `write_rows`
    of `tensor` ([2 * slots + 2, ...]); the manager swaps them at commit."""

    tensor: torch.Tensor
    read_rows: torch.Tensor  # [R] int32
    write_rows: torch.Tensor  # [R] int32
