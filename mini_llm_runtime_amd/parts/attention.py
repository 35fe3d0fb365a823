"""Attention mixers."""

from __future__ import annotations

import math
from typing import Optional

import torch

from ..cache.spec import PagedKVSpec
from ..kernels.limits import check_attention_sizes
from .base import Mixer, Part, PositionEncoding
from .context import MixerPlan, PlanInput, StepContext
from .registry import build_part, register_part
from .spec import ParamSpec, PartSpec


@register_part("mixer", "gqa_attention")
class GQAAttention(Mixer):
    """Grouped-query causal self-attention over the paged cache.

    Order of work, from src/mini_llm_runtime/qwen_model_runner.py:75-183: project
    q, k, v (with bias when `qkv_bias`), encode positions into q and k, store the
    encoded k and the raw v in the cache, attend, merge heads, project out.  Query
    head h reads KV head h // (num_heads // num_kv_heads) (:64-72).  Scores are
    scaled by `scale` (default head_dim^-0.5, :157) and a query at position p sees
    the keys 0..p of its own request (:158-175), or only the last `window` of
    them.  Unlike the reference, which runs whole prompts from in-flight tensors
    and single tokens from the pages, every query here reads the pages, after the
    step's own keys were written: a prompt portion and a decoded token are the
    same case.

    The three projections are one matrix product over the row-wise concatenation
    [Wq; Wk; Wv] (made by the weight rules at load time).
    """

    replayable = True
    takes_pending_norm = True  # `h` goes to the query/key/value product only

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        position: Optional[PartSpec] = None,
        qkv_bias: bool = True,
        o_bias: bool = False,
        window: Optional[int] = None,
        scale: Optional[float] = None,
    ) -> None:
        if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
            raise ValueError("num_heads must be a positive multiple of num_kv_heads")
        if head_dim <= 0:
            raise ValueError("head_dim must be > 0")
        check_attention_sizes(num_heads, num_kv_heads, head_dim)  # refused here, not at the first step
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.qkv_bias = bool(qkv_bias)
        self.o_bias = bool(o_bias)
        self.window = None if window is None else int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.position: Optional[PositionEncoding] = (
            build_part("position", position) if position is not None else None
        )
        self.qkv_weight: Optional[torch.Tensor] = None
        self.qkv_bias_vec: Optional[torch.Tensor] = None
        self.o_weight: Optional[torch.Tensor] = None
        self.o_bias_vec: Optional[torch.Tensor] = None

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    def param_specs(self) -> dict[str, ParamSpec]:
        width = self.q_size + 2 * self.kv_size
        specs = {
            "qkv_weight": ParamSpec((width, self.hidden_size)),
            "o_weight": ParamSpec((self.hidden_size, self.q_size)),
        }
        if self.qkv_bias:
            specs["qkv_bias_vec"] = ParamSpec((width,), keep_stored_precision=True)
        if self.o_bias:
            specs["o_bias_vec"] = ParamSpec((self.hidden_size,), keep_stored_precision=True)
        return specs

    def children(self) -> dict[str, Part]:
        return {"position": self.position} if self.position is not None else {}

    def cache_spec(self) -> PagedKVSpec:
        return PagedKVSpec(self.num_kv_heads, self.head_dim, self.window)

    def plan(self, ops, shape: PlanInput) -> Optional[MixerPlan]:
        make = getattr(ops, "attention_plan", None)  # the kernel library knows what its kernels want
        return make(shape) if make is not None else None

    def forward(self, ctx: StepContext, h: torch.Tensor, site: int) -> torch.Tensor:
        ops = ctx.ops
        cache = ctx.kv(site)
        rotation = self.position.rotation(ctx) if self.position is not None else None
        pages = dict(
            num_heads=self.num_heads,
            num_kv_heads=self.num_kv_heads,
            head_dim=self.head_dim,
            block_size=cache.block_size,
            write=cache.writable,
        )
        if self.position is not None and rotation is None:
            # a position encoding with a rule of its own: it sees the queries and keys between
            # the product and the cache write
            qkv = ops.linear(h, self.qkv_weight, self.qkv_bias_vec)
            tokens = qkv.shape[0]
            q = qkv[:, : self.q_size].view(tokens, self.num_heads, self.head_dim)
            k = qkv[:, self.q_size : self.q_size + self.kv_size].view(tokens, self.num_kv_heads, self.head_dim)
            self.position.apply(ctx, q, k)
            ops.rope_kv_write(qkv, None, cache.slot_mapping, cache.key, cache.value, **pages)
        else:
            qkv = ops.qkv_rope_write(
                h, self.qkv_weight, self.qkv_bias_vec, rotation, cache.slot_mapping, cache.key, cache.value, **pages
            )
        if cache.writable:
            cache.written()
        cache.reading()
        attended = ops.paged_attention(
            qkv,
            cache.key,
            cache.value,
            cache.block_table,
            ctx,
            num_heads=self.num_heads,
            num_kv_heads=self.num_kv_heads,
            head_dim=self.head_dim,
            block_size=cache.block_size,
            scale=self.scale,
            window=self.window,
            defer_merge=True,  # the output product is the only reader
            plan=ctx.plan(getattr(ops, "ATTENTION_PLAN", None)),
        )
        return ops.linear(attended, self.o_weight, self.o_bias_vec, for_stream=True)  # the next norm's delta
