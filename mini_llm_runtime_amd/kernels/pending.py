"""Activations that have not been computed yet, handed from one operation to the next so
that the consumer can compute them inside its own kernel.

A decode step of a small model is bound by its number of dependent kernels.  A norm followed
by a matrix product, and the merge of the decode attention's partitions followed by the
output product, are each one kernel when the product makes its activations itself; whether
it can is for the kernel library to say (few tokens, a width that fits LDS).  Either way the
consumer ends up with the same values as if the producer had run on its own.

A third link goes away at the other end of a part: its last product (the output projection, the
down projection) is followed by "add to the residual stream, then norm".  When that product is
handed on unrun (`PendingLinear`), the norm behind it can run it as a kernel that owns whole
output columns, adds them to the stream itself, and leaves the norm's activations short of one
factor per row (`PendingScale`), which the product that consumes them applies to its sums.
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


@dataclass
class PendingLinear:
    """x W^T + b that has not run: a part's output on its way into the residual stream.  The norm
    that receives it as its delta runs it, together with the addition, where the kernel library can;
    anything else that needs the values settles it into a tensor first."""

    x: object  # [T, K] in the engine's dtype, or a PendingMerge
    weight: torch.Tensor  # [N, K]
    bias: Optional[torch.Tensor]

    @property
    def shape(self) -> tuple[int, int]:
        return (self.x.shape[0], self.weight.shape[0])


@dataclass
class PendingScale:
    """RMSNorm(stream) * weight short of its division by the root mean square: `h` = weight *
    stream in the engine's dtype, `sumsq` [T, parts] float32 partial sums of squares of every
    stream row.  A product that consumes it multiplies the sums of row t by
    rsqrt(sum(sumsq[t]) / width + eps).  `residual` is the stream (already updated)."""

    h: torch.Tensor
    sumsq: torch.Tensor
    weight: torch.Tensor
    eps: float
    residual: torch.Tensor
    value: Optional[torch.Tensor] = None  # the normed activations, once a norm kernel of its own made them

    @property
    def shape(self) -> torch.Size:
        return self.h.shape
