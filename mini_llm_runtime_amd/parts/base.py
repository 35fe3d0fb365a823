"""Interfaces of the parts a layer is put together from.

A part is constructed from sizes and constants only, declares its parameters
(`param_specs`) and, for mixers, what it needs of the cache (`cache_spec`).
`bind` hands it the loaded tensors.  `forward` computes on token-major
activations [T, width] for whatever batch the `StepContext` describes.
"""

from __future__ import annotations

from typing import Any, Mapping, Optional

import torch

from .context import MixerPlan, PlanInput, StepContext
from .spec import ParamSpec


class Part:
    # True when `forward` does nothing on the host that depends on the step's DATA (which
    # requests, their lengths, token values): everything of that kind is read on the device from
    # the tensors of the `StepContext`, and the host only uses the context's sizes (tokens,
    # entries, tiles, block table width).  A step of such parts can be recorded as a HIP graph
    # and replayed for later steps of the same sizes.  Off by default: a part has to say so.
    replayable = False
    # A mixer or feed-forward that hands its input `h` to `ops.linear` / `ops.qkv_rope_write`
    # and to nothing else may say so: it then may receive a norm that has not run yet (which
    # those operations run, fused into their own kernel where they can) instead of a tensor.
    takes_pending_norm = False
    # False for a part that needs a request's whole prompt in one step (it cannot go on from a
    # cached prefix): the scheduler then never cuts prompts of a model that holds it.
    splittable = True

    def param_specs(self) -> dict[str, ParamSpec]:
        return {}

    def bind(self, params: Mapping[str, torch.Tensor], *, dtype: torch.dtype, device: torch.device) -> None:
        """Receive the loaded parameters (keys of `param_specs`)."""
        for name, tensor in params.items():
            setattr(self, name, tensor)

    def children(self) -> dict[str, "Part"]:
        """Parts nested inside this one (their parameters live under `<name>.`)."""
        return {}


class Norm(Part):
    # True when `forward` takes `defer=True` and may then return a pending norm (an object with a
    # `residual` attribute that holds the updated stream once a consumer has run it).
    can_defer = False

    def forward(self, ctx: StepContext, x: torch.Tensor, delta: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x: float32 residual stream [T, H].  When `delta` is given, first x += delta
        (in place, summed in 32-bit); returns norm(x) in the engine's dtype.  `delta` is a
        part's output: [T, H] in the engine's dtype, or, from a part that ends in
        `ops.linear(..., for_stream=True)`, whatever that returned (a float32 stack [S, T, H] whose
        sum over S it is, or a product that has not run): the kernel library's norm takes all of them."""
        raise NotImplementedError


class PositionEncoding(Part):
    def rotation(self, ctx: StepContext) -> Optional[tuple[torch.Tensor, torch.Tensor, int]]:
        """(cos [T, r/2], sin [T, r/2], r) when the encoding is a half-split rotation of
        the first r dims of every head that the fused kernel can apply; else None and
        `apply` is called instead."""
        return None

    def apply(self, ctx: StepContext, q: torch.Tensor, k: torch.Tensor) -> None:
        """Encode positions into q [T, Hq, d] and k [T, Hkv, d] in place."""
        raise NotImplementedError

    def embed(self, ctx: StepContext) -> torch.Tensor:
        """[T, hidden] (float32 or the engine's dtype) to be added to the embedded tokens, for an
        encoding that a model names as its `position_embedding`."""
        raise NotImplementedError


class Mixer(Part):
    def cache_spec(self) -> Any:
        """PagedKVSpec, SlotStateSpec or None."""
        return None

    def plan(self, ops: Any, shape: PlanInput) -> Optional[MixerPlan]:
        """What this mixer's kernels need planned on the host for a step of this shape (tiles,
        counts, launch sizes), or None.  The step function uploads the plan's arrays with the
        step's metadata, hands the plan to `forward` through `ctx.plan(key)`, and records a
        step only for replay under plans of the same sizes; it knows nothing of what is in it.
        A mixer that plans does so for every shape, always under the same key; of several mixers
        with the same key the first one's plan is used (they make the same plan from a shape)."""
        return None

    def forward(self, ctx: StepContext, h: torch.Tensor, site: int) -> torch.Tensor:
        """h: normed activations [T, H] in the engine's dtype; returns [T, H]."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx: StepContext, h: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """An arrangement of a mixer, a feed-forward and norms around the residual stream."""

    def forward(
        self, ctx: StepContext, x: torch.Tensor, delta: Optional[torch.Tensor], site: int
    ) -> tuple[torch.Tensor, Optional[torch.Tensor]]:
        """x: float32 residual stream.  `delta` is the previous layer's output that has
        not been added yet (None at the first layer).  Returns the residual stream (the
        same tensor updated in place, or a new one) and this layer's own not-yet-added
        output."""
        raise NotImplementedError
