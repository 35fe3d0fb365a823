"""A norm that has not been computed yet.

A block hands `DeferredNorm(x, delta, weight, eps)` to a part instead of the
normed activations.  A part that starts with a matrix product passes it straight
to `ops.linear`, which may fuse "x += delta, norm" into that product's kernel (one
kernel instead of two, which matters when a decode step is a chain of very short
kernels); anything else calls `tensor()` and gets the activations computed the
plain way.  Either way `residual` is the updated residual stream afterwards.
"""

from __future__ import annotations

from typing import Any, Optional

import torch


class DeferredNorm:
    def __init__(self, ops: Any, x: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float) -> None:
        self.ops = ops
        self.weight = weight
        self.eps = float(eps)
        self._x = x
        self._delta = delta
        self._tensor: Optional[torch.Tensor] = None
        self._added = delta is None

    @property
    def materialized(self) -> bool:
        return self._tensor is not None

    @property
    def shape(self) -> torch.Size:
        return self._x.shape

    def inputs(self) -> tuple[torch.Tensor, Optional[torch.Tensor]]:
        """(residual stream, delta still to be added) for a kernel that fuses the norm."""
        return self._x, (None if self._added else self._delta)

    def fused(self, x_out: Optional[torch.Tensor]) -> None:
        """A fused kernel consumed the norm and wrote x + delta to `x_out`."""
        if not self._added and self._delta is not None:
            if x_out is None:
                raise RuntimeError("a fused norm with a delta must write the summed residual stream")
            self._x = x_out
        self._added = True

    def tensor(self) -> torch.Tensor:
        """The normed activations, computed now if they were not yet (adds delta in place)."""
        if self._tensor is None:
            delta = None if self._added else self._delta
            self._tensor = self.ops.rmsnorm(self._x, self.weight, self.eps, delta=delta)
            self._added = True
        return self._tensor

    @property
    def residual(self) -> torch.Tensor:
        """The residual stream including delta; computes the addition if nobody has."""
        if not self._added:
            if self._delta is not None:
                self.ops.add_(self._x, self._delta)
            self._added = True
        return self._x
