"""Position encodings."""

from __future__ import annotations

from typing import Mapping, Optional

import numpy as np
import torch

from .base import PositionEncoding
from .context import StepContext
from .registry import register_part


@register_part("position", "rotary")
class RotaryEmbedding(PositionEncoding):
    """Half-split rotary encoding: dims j and j + r/2 of a head are rotated by the
    angle `pos * theta^(-2j/r)`.

    Formula: src/mini_llm_runtime/qwen_model_runner.py:34-61 (`rotate_half` pairs the
    two halves; the reference rotates the whole head, r = head_dim).  The inverse
    frequencies are computed once in float64 on the host; the angles and their
    cosines and sines are computed once per step for all layers that share this
    encoding's constants.
    """

    replayable = True


    def __init__(self, head_dim: int, theta: float, rotary_dim: Optional[int] = None) -> None:
        rotary_dim = head_dim if rotary_dim is None else int(rotary_dim)
        if rotary_dim <= 0 or rotary_dim % 2 or rotary_dim > head_dim:
            raise ValueError("rotary_dim must be even and within head_dim")
        if not theta > 0:
            raise ValueError("theta must be > 0")
        self.head_dim = int(head_dim)
        self.rotary_dim = rotary_dim
        self.theta = float(theta)
        exponents = np.arange(0, rotary_dim, 2, dtype=np.float64) / rotary_dim
        self._inv_freq_host = 1.0 / (self.theta**exponents)
        self.inv_freq: Optional[torch.Tensor] = None

    def bind(self, params: Mapping[str, torch.Tensor], *, dtype: torch.dtype, device: torch.device) -> None:
        self.inv_freq = torch.from_numpy(self._inv_freq_host).to(device)

    def rotation(self, ctx: StepContext):
        key = ("rotary", self.rotary_dim, self.theta)
        if key not in ctx.memo:
            cos, sin = ctx.ops.rope_table(ctx.positions, self.inv_freq)
            ctx.memo[key] = (cos, sin, self.rotary_dim)
        return ctx.memo[key]


@register_part("position", "none")
class NoPosition(PositionEncoding):
    """No position encoding at all (order enters through the causal mask only)."""

    replayable = True


    def __init__(self, head_dim: int = 0) -> None:
        self.head_dim = head_dim

    def apply(self, ctx: StepContext, q: torch.Tensor, k: torch.Tensor) -> None:
        return None
