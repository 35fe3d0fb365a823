"""A decoder-only model put together from a `ModelSpec`.

The model owns the embedding table, the layers (blocks of parts), the final norm
and the output head, and runs the execution sites in the order the spec lists.
It holds no sizes of its own: everything comes from the spec.
"""

from __future__ import annotations

from typing import Iterator, Mapping, Optional

import torch

from .base import Block, Part
from .context import StepContext
from .registry import build_part
from .spec import LayerSpec, ModelSpec, ParamSpec, PartSpec


def _build_layer(spec: LayerSpec) -> Block:
    mixer = build_part("mixer", spec.mixer)
    feed_forward = build_part("feed_forward", spec.feed_forward)
    norms = {name: build_part("norm", s) for name, s in spec.norms.items()}
    return build_part("block", PartSpec(spec.block), mixer=mixer, feed_forward=feed_forward, norms=norms)


def _walk(prefix: str, part: Part) -> Iterator[tuple[str, Part]]:
    yield prefix, part
    for name, child in part.children().items():
        yield from _walk(f"{prefix}.{name}", child)


class DecoderModel:
    def __init__(self, spec: ModelSpec) -> None:
        self.spec = spec
        self.layers: list[Block] = [_build_layer(s) for s in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm)
        self.position_embedding = (
            build_part("position", spec.position_embedding) if spec.position_embedding is not None else None
        )
        self.embed_weight: Optional[torch.Tensor] = None
        self.head_weight: Optional[torch.Tensor] = None
        self.head_bias: Optional[torch.Tensor] = None
        self.dtype: Optional[torch.dtype] = None
        self.device: Optional[torch.device] = None
        if not spec.order:
            raise ValueError("the execution order is empty")
        specs = []
        for site, entry in enumerate(spec.order):
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(f"order entry {site} names layer {entry.layer}, the model has {len(self.layers)}")
            own = self.layers[entry.layer].mixer.cache_spec()
            if entry.reads_cache_of is not None:
                src = entry.reads_cache_of
                if not 0 <= src < site or spec.order[src].reads_cache_of is not None:
                    raise ValueError(f"order entry {site} must read the cache of an earlier site that owns one")
                if specs[src] != own:
                    raise ValueError(f"order entry {site} reads a cache of another shape than its mixer needs")
            specs.append(own)
        self._site_needs = specs

    # ---- structure --------------------------------------------------------------------
    @property
    def num_sites(self) -> int:
        return len(self.spec.order)

    def site_cache_specs(self) -> list[Optional[object]]:
        """For every execution site the cache it owns (None: it owns none)."""
        out: list[Optional[object]] = []
        for site, entry in enumerate(self.spec.order):
            out.append(None if entry.reads_cache_of is not None else self._site_needs[site])
        return out

    def cache_site_of(self, site: int) -> int:
        src = self.spec.order[site].reads_cache_of
        return site if src is None else src

    @property
    def replayable(self) -> bool:
        """Every part says that its steps can be recorded and replayed (`Part.replayable`)."""
        return all(part.replayable for _, part in self.named_parts())

    @property
    def splittable(self) -> bool:
        """Every part can go on from a cached prefix, so prompts may be cut into portions."""
        return all(part.splittable for _, part in self.named_parts())

    def named_parts(self) -> Iterator[tuple[str, Part]]:
        for i, layer in enumerate(self.layers):
            yield from _walk(f"layers.{i}", layer)
        yield from _walk("final_norm", self.final_norm)
        if self.position_embedding is not None:
            yield from _walk("position_embedding", self.position_embedding)

    def param_specs(self) -> dict[str, ParamSpec]:
        specs: dict[str, ParamSpec] = {
            "embed.weight": ParamSpec((self.spec.vocab_size, self.spec.hidden_size)),
        }
        if not self.spec.tie_word_embeddings:
            specs["head.weight"] = ParamSpec((self.spec.vocab_size, self.spec.hidden_size))
        if self.spec.head_bias:
            specs["head.bias"] = ParamSpec((self.spec.vocab_size,), keep_stored_precision=True)
        for path, part in self.named_parts():
            for name, p in part.param_specs().items():
                specs[f"{path}.{name}"] = p
        return specs

    def bind(self, params: Mapping[str, torch.Tensor], *, dtype: torch.dtype, device: torch.device) -> None:
        expected = set(self.param_specs())
        if set(params) != expected:
            raise ValueError(
                f"bind: parameters do not match: missing {sorted(expected - set(params))}, "
                f"unexpected {sorted(set(params) - expected)}"
            )
        self.dtype = dtype
        self.device = torch.device(device)
        self.embed_weight = params["embed.weight"]
        self.head_weight = params["embed.weight"] if self.spec.tie_word_embeddings else params["head.weight"]
        self.head_bias = params.get("head.bias")
        for path, part in self.named_parts():
            own = {name: params[f"{path}.{name}"] for name in part.param_specs()}
            part.bind(own, dtype=dtype, device=self.device)

    def weight_bytes(self) -> int:
        seen: dict[int, int] = {}
        tensors = [self.embed_weight, self.head_weight, self.head_bias]
        for _, part in self.named_parts():
            tensors.extend(getattr(part, name) for name in part.param_specs())
        for t in tensors:
            if t is not None:
                seen[t.data_ptr()] = t.numel() * t.element_size()
        return sum(seen.values())

    # ---- compute ----------------------------------------------------------------------
    def forward(
        self,
        ctx: StepContext,
        logit_rows: Optional[torch.Tensor],
        site_outputs: Optional[list] = None,
    ) -> Optional[torch.Tensor]:
        """Run the step's tokens through all sites; logits [K, vocab] float32 at `logit_rows`.

        site_outputs: a list that receives, after every site, the float32 residual stream at
        `logit_rows` ([K, hidden]): what the reference's `return_layer_outputs` captures
        after each layer (src/mini_llm_runtime/qwen_model_runner.py:266-281).  A tool for
        finding the layer at which a wrong logit first appears; it adds a few small kernels
        per site and is never recorded into a graph."""
        ops = ctx.ops
        spec = self.spec
        x = ops.embedding(self.embed_weight, ctx.token_ids)
        if spec.embedding_scale != 1.0:
            ops.scale_softcap_(x, spec.embedding_scale)
        if self.position_embedding is not None:
            ops.add_(x, self.position_embedding.embed(ctx))
        delta: Optional[torch.Tensor] = None
        capture = site_outputs is not None and logit_rows is not None and logit_rows.numel() > 0
        for site, entry in enumerate(self.spec.order):
            x, delta = self.layers[entry.layer].forward(ctx, x, delta, site)
            if capture:
                # the site's own output is not added into the stream yet: add it here, in 32-bit
                rows = ops.gather_rows(x, logit_rows)
                if delta is not None:
                    own = ops.gather_rows(delta, logit_rows)
                    own = getattr(ops, "settle", lambda t: t)(own)  # a product that has not run yet, run now
                    rows = rows + (own.sum(0) if own.dim() == 3 else own.float())
                site_outputs.append(rows)
        if logit_rows is None or logit_rows.numel() == 0:
            return None
        if ctx.logits_for_all:
            rows, delta_rows = x, delta
        else:
            rows = ops.gather_rows(x, logit_rows)
            delta_rows = ops.gather_rows(delta, logit_rows) if delta is not None else None
        # the head is a product like any other: it may take a norm that has not run
        if self.final_norm.can_defer:
            h = self.final_norm.forward(ctx, rows, delta_rows, defer=True)
        else:
            h = self.final_norm.forward(ctx, rows, delta_rows)
        logits = ops.linear(h, self.head_weight, self.head_bias, out_dtype=torch.float32)
        if spec.logit_scale != 1.0 or spec.logit_softcap is not None:
            ops.scale_softcap_(logits, spec.logit_scale, spec.logit_softcap)
        return logits
