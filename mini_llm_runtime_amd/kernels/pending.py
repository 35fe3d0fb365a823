"""Activations that have not been computed yet, handed from one operation to the next so
that the consumer can compute them inside its own kernel.

A decode step of a small model is bound by its number of dependent kernels.  A norm followed
by a matrix product, and the merge of the decode attention's partitions followed by the
output product, are each one kernel when the product makes its activations itself; whether
it can is for the kernel library to say (few tokens, a width that fits LDS).  Either way the
consumer ends up with the same values as if the producer had run on its own.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch


@dataclass
class PendingNorm:
    """RMSNorm(x + delta) * weight that has not run.  Whoever runs it (fused into a product,
    or as a kernel of its own) leaves the updated residual stream in `residual`."""

    x: torch.Tensor  # float32 [T, H]
    delta: Optional[torch.Tensor]  # [T, H] in the engine's dtype, or float32 [S, T, H], or None
    weight: torch.Tensor
    eps: float
    residual: Optional[torch.Tensor] = None
    value: Optional[torch.Tensor] = None  # the normed activations, once a kernel of its own made them

    @property
    def shape(self) -> torch.Size:
        return self.x.shape


@dataclass
class PendingMerge:
    """The decode attention's output [T, heads * head_dim] still in partitions
    ([T, heads, splits, head_dim + 2] float32: numerator, base-2 maximum, denominator)."""

    partial: torch.Tensor
    cu_q: torch.Tensor
    context_lens: torch.Tensor
    tokens: int
    heads: int
    head_dim: int
    window: int
    part: int
    splits: int
    library: object  # the attention library that can merge them on its own

    @property
    def shape(self) -> tuple[int, int]:
        return (self.tokens, self.heads * self.head_dim)
