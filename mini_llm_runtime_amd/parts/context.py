"""What a part sees of a step: the tokens of the batch, where they sit in their
requests, and handles to the cache of the execution site it runs at.  It is the
same for every mixer kind; nothing in it names a model.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Optional

import numpy as np
import torch

@dataclass(frozen=True)
class PlanInput:
    """What a mixer may look at when it plans its kernels for a step: the new tokens and the
    cached tokens of every entry, and a bound on the entries' contexts after the step (the
    exact maximum, or, for a step that is being recorded, the capacity of its block tables)."""

    q_lens: np.ndarray  # [R] tokens of this step
    q_starts: np.ndarray  # [R] tokens cached before it
    max_context: int


@dataclass
class MixerPlan:
    """A mixer's launch plan for one step.  `arrays` (int32) are uploaded with the step's other
    metadata; `sizes` are what the mixer's host code needs to launch (grid sizes, counts): they
    are part of a recorded step's identity, so a recording is only replayed for steps whose
    plans have the same sizes.  Mixers whose plans have the same `key` share one plan."""

    key: Any
    arrays: dict  # name -> np.ndarray (int32)
    sizes: dict  # name -> int


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
    host: Any  # the StepLayout (numpy arrays) for parts that work on the host; None while a step is recorded
    logits_for_all: bool = False  # the wanted rows are all tokens, in order: no gather needed
    kv_views: dict[int, KVView] = field(default_factory=dict)
    state_views: dict[int, StateView] = field(default_factory=dict)
    plans: dict[Any, Any] = field(default_factory=dict)  # MixerPlan.key -> its sizes and device arrays, as attributes
    memo: dict[Any, Any] = field(default_factory=dict)

    def plan(self, key: Any) -> Any:
        """The plan some mixer made under `key` (None: none did): an object whose attributes are
        the plan's sizes and, as device tensors, its arrays."""
        return self.plans.get(key)

    def kv(self, site: int) -> KVView:
        return self.kv_views[site]

    def state(self, site: int) -> StateView:
        return self.state_views[site]
