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
    matrix product over a matrix that holds the rows of Wgate and Wup woven in pairs
    (gate 0, gate 1, up 0, up 1, gate 2, ...; made by the weight rules), and
    silu(gate) * up is that product's epilogue.
    """

    replayable = True
    takes_pending_norm = True  # `h` goes to the gate/up product only

    def __init__(self, hidden_size: int, intermediate_size: int) -> None:
        if hidden_size <= 0 or intermediate_size <= 0 or intermediate_size % 2:
            raise ValueError("SwiGLU sizes must be > 0 and the intermediate size even")
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
        hidden = ops.linear(h, self.gate_up_weight, None, swiglu=True)
        return ops.linear(hidden, self.down_weight, None, for_stream=True)  # the next norm's delta
