"""Arrangements of parts around the residual stream."""

from __future__ import annotations

from typing import Mapping, Optional

import torch

from .base import Block, FeedForward, Mixer, Norm, Part
from .context import StepContext
from .registry import register_part


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    """x += mixer(norm_in(x)); x += feed_forward(norm_post(x)).

    src/mini_llm_runtime/qwen_model_runner.py:198-218.  The residual stream is kept
    in 32-bit; each addition is fused into the norm that follows it, so the block
    hands its last output to the next block (or the model) un-added.
    """

    replayable = True


    norm_names = ("input", "post_mixer")

    def __init__(self, mixer: Mixer, feed_forward: FeedForward, norms: Mapping[str, Norm]) -> None:
        missing = [n for n in self.norm_names if n not in norms]
        if missing:
            raise ValueError(f"pre_norm block needs the norms {self.norm_names}, missing {missing}")
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norm_input = norms["input"]
        self.norm_post_mixer = norms["post_mixer"]

    def children(self) -> dict[str, Part]:
        return {
            "mixer": self.mixer,
            "feed_forward": self.feed_forward,
            "norm_input": self.norm_input,
            "norm_post_mixer": self.norm_post_mixer,
        }

    def forward(
        self, ctx: StepContext, x: torch.Tensor, delta: Optional[torch.Tensor], site: int
    ) -> tuple[torch.Tensor, Optional[torch.Tensor]]:
        h = self.norm_input.forward(ctx, x, delta)
        mixed = self.mixer.forward(ctx, h, site)
        h = self.norm_post_mixer.forward(ctx, x, mixed)
        return x, self.feed_forward.forward(ctx, h)
