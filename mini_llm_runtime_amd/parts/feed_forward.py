"""Feed-forward parts."""

from __future__ import annotations

from typing import Optional

import torch

from .base import FeedForward
from .context import StepContext
from .registry import register_part
from .spec import ParamSpec


@register_part("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    """Dense gated feed-forward: `down(silu(gate(x)) * up(x))`, no biases.

    Formula: src/mini_llm_runtime/qwen_model_runner.py:215-217.  Gate and up are one
    matrix product over [Wgate; Wup] (concatenated by the weight rules).
    """

    def __init__(self, hidden_size: int, intermediate_size: int) -> None:
        if hidden_size <= 0 or intermediate_size <= 0:
            raise ValueError("SwiGLU sizes must be > 0")
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.gate_up_weight: Optional[torch.Tensor] = None
        self.down_weight: Optional[torch.Tensor] = None

    def param_specs(self) -> dict[str, ParamSpec]:
        return {
            "gate_up_weight": ParamSpec((2 * self.intermediate_size, self.hidden_size)),
            "down_weight": ParamSpec((self.hidden_size, self.intermediate_size)),
        }

    def forward(self, ctx: StepContext, h: torch.Tensor) -> torch.Tensor:
        ops = ctx.ops
        gate_up = ops.linear(h, self.gate_up_weight, None)
        hidden = ops.silu_mul(gate_up)
        return ops.linear(hidden, self.down_weight, None)
