"""Norms."""

from __future__ import annotations

from typing import Optional

import torch

from .base import Norm
from .context import StepContext
from .registry import register_part
from .spec import ParamSpec


@register_part("norm", "rms_norm")
class RMSNorm(Norm):
    """`weight * x * rsqrt(mean(x^2) + eps)`: no centring, no bias, weight used as is.

    Formula: src/mini_llm_runtime/qwen_model_runner.py:22-26.  Statistics and the
    scaling are computed in 32-bit from the 32-bit residual stream; the result is
    rounded once to the engine's dtype.
    """

    replayable = True
    can_defer = True

    def __init__(self, size: int, eps: float) -> None:
        if size <= 0 or not eps >= 0:
            raise ValueError("RMSNorm needs size > 0 and eps >= 0")
        self.size = int(size)
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.size,), init="one_plus_normal", keep_stored_precision=True)}

    def forward(self, ctx: StepContext, x: torch.Tensor, delta: Optional[torch.Tensor] = None, defer: bool = False):
        """defer: the consumer takes a norm that has not run (see `Part.takes_pending_norm`); the
        kernel library decides whether there is something to gain."""
        if defer:
            make = getattr(ctx.ops, "defer_norm", None)
            pending = make(x, self.weight, self.eps, delta) if make is not None else None
            if pending is not None:
                return pending
        return ctx.ops.rmsnorm(x, self.weight, self.eps, delta=delta)

