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
        h = _norm(self.norm_input, self.mixer, ctx, x, delta)
        mixed = self.mixer.forward(ctx, h, site)
        x = _stream_after(h, x)
        h = _norm(self.norm_post_mixer, self.feed_forward, ctx, x, mixed)
        out = self.feed_forward.forward(ctx, h)
        return _stream_after(h, x), out


def _norm(norm: Norm, consumer: Part, ctx: StepContext, x: torch.Tensor, delta: Optional[torch.Tensor]):
    """norm(x + delta) for `consumer`: possibly not run yet, if both sides can deal with that."""
    if norm.can_defer and consumer.takes_pending_norm:
        return norm.forward(ctx, x, delta, defer=True)
    return norm.forward(ctx, x, delta)


def _stream_after(h, x: torch.Tensor) -> torch.Tensor:
    """The residual stream once `h` was consumed: the tensor the norm updated in place, or the
    new one that the consumer of a pending norm wrote."""
    if isinstance(h, torch.Tensor):
        return x
    if h.residual is None:
        raise RuntimeError("a part that takes pending norms did not hand its input to an operation that runs them")
    return h.residual
