"""What a part sees of a step: the tokens of the batch, where they sit in their
requests, and handles to the cache of the execution site it runs at.  It is the
same for every mixer kind; nothing in it names a model.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Optional

import numpy as np
import torch

from ..cache.views import KVView, StateView  # noqa: F401  (part of this module's surface)


@dataclass(frozen=True)
class PlanInput:
    """What a mixer may look at when it plans its kernels for a step: the new tokens and the
    cached tokens of every entry, and a bound on the entries' contexts after the step (the
    exact maximum, or, for a step that is being recorded, the capacity of its block tables)."""

    q_lens: np.ndarray  # [R] tokens of this step
    q_starts: np.ndarray  # [R] tokens cached before it
    max_context: int
    # The step itself, for plans that need more than its shape: the cache manager's `StepLayout` (host
    # arrays: request ids and slots, positions, block tables and slot mappings per pool, state rows) and
    # the token ids.  Both are None when only a shape exists (the probe when a runner is built).  For a
    # recorded step of single tokens, padded to a power of two, they describe the real entries while
    # q_lens and q_starts are padded.
    layout: Any = None
    token_ids: Optional[np.ndarray] = None


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
    site_views: dict[int, Any] = field(default_factory=dict)  # execution site -> what its cache spec made for this step
    plans: dict[Any, Any] = field(default_factory=dict)  # MixerPlan.key -> its sizes and device arrays, as attributes
    memo: dict[Any, Any] = field(default_factory=dict)

    def plan(self, key: Any) -> Any:
        """The plan some mixer made under `key` (None: none did): an object whose attributes are
        the plan's sizes and, as device tensors, its arrays."""
        return self.plans.get(key)

    def cache(self, site: int) -> Any:
        """The view of the cache that execution site `site` uses in this step, as its spec made it."""
        return self.site_views[site]

    def kv(self, site: int) -> KVView:
        return self.site_views[site]

    def state(self, site: int) -> StateView:
        return self.site_views[site]

    # the views by the names they had when there were two kinds
    @property
    def kv_views(self) -> dict[int, Any]:
        return self.site_views

    @property
    def state_views(self) -> dict[int, Any]:
        return self.site_views
