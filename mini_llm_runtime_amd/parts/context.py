"""What a part sees of a step: the tokens of the batch, where they sit in their
requests, and handles to the cache of the execution site it runs at.  It is the
same for every mixer kind; nothing in it names a model.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Optional

import numpy as np
import torch

QUERY_TILE = 64  # queries of one request that a mixer's prompt kernel takes together


def query_tiles(q_lens, q_starts=None) -> np.ndarray:
    """[num_tiles, 2] int32 (entry, first query) covering every entry with more than one new
    token, the tiles with the most keys before them first: a kernel that hands them to the
    compute units in that order can start the heavy ones early and pair them with light ones."""
    tiles = [(r, q0) for r, n in enumerate(q_lens) if n > 1 for q0 in range(0, int(n), QUERY_TILE)]
    if q_starts is None:
        q_starts = [0] * len(q_lens)
    tiles.sort(key=lambda t: -(int(q_starts[t[0]]) + t[1]))
    return np.asarray(tiles, dtype=np.int32).reshape(-1, 2)


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
    of `tensor` ([2 * slots, ...]); the manager swaps them at commit."""

    tensor: torch.Tensor
    read_rows: torch.Tensor  # [R] int32
    write_rows: torch.Tensor  # [R] int32


@dataclass
class StepContext:
    ops: Any
    dtype: torch.dtype
    device: torch.device
    num_tokens: int
    num_entries: int
    token_ids: torch.Tensor  # [T] int32
    positions: torch.Tensor  # [T] int32 absolute position of each token in its request
    token_entry: torch.Tensor  # [T] int32 entry index of each token
    cu_q: torch.Tensor  # [R+1] int32 first token of each entry
    q_starts: torch.Tensor  # [R] int32 tokens cached before this step
    context_lens: torch.Tensor  # [R] int32 tokens visible after this step's write
    max_q_len: int
    max_context_len: int
    host: Any  # the StepLayout (numpy arrays) for parts that plan on the host
    # plan for attention kernels: tiles of 64 queries over entries with several new
    # tokens ([num_tiles, 2]: entry, first query), and the single-token entries
    query_tiles: Optional[torch.Tensor] = None
    num_query_tiles: int = 0
    num_decode_entries: int = 0
    max_decode_context: int = 0
    logits_for_all: bool = False  # the wanted rows are all tokens, in order: no gather needed
    kv_views: dict[int, KVView] = field(default_factory=dict)
    state_views: dict[int, StateView] = field(default_factory=dict)
    memo: dict[Any, Any] = field(default_factory=dict)

    def kv(self, site: int) -> KVView:
        return self.kv_views[site]

    def state(self, site: int) -> StateView:
        return self.state_views[site]
