"""Data that describes a model: which parts each layer is made of, with which
sizes, in which order the layers run, and which checkpoint tensor feeds which
parameter.  Nothing here computes; builders in `models/` produce these objects
from a typed configuration and `parts.model.DecoderModel` turns them into code.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional


@dataclass(frozen=True)
class ParamSpec:
    """One parameter tensor of a part.

    init: "normal" (N(0, std)) or "one_plus_normal" (1 + N(0, std)); used by the
        random-weights mode only.
    keep_stored_precision: a vector (norm weight, bias) that a checkpoint stores in
        32-bit stays 32-bit in the bfloat16 engine; matrices always take the
        engine's dtype.
    """

    shape: tuple[int, ...]
    init: str = "normal"
    keep_stored_precision: bool = False


@dataclass(frozen=True)
class PartSpec:
    """A part chosen by kind name, with its constructor arguments."""

    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: an arrangement (`block`) of a mixer, a feed-forward and norms."""

    block: str
    mixer: PartSpec
    feed_forward: PartSpec
    norms: Mapping[str, PartSpec]


@dataclass(frozen=True)
class OrderEntry:
    """One execution site: run `layer`; `reads_cache_of` names an earlier site whose
    cache this site reads instead of owning one (None: the site owns its cache)."""

    layer: int
    reads_cache_of: Optional[int] = None


@dataclass(frozen=True)
class WeightRule:
    """Checkpoint tensor `name` fills rows [row_start, row_start + rows) of parameter
    `dest` (all of it when `rows` is None).  With `block` and `period` the rows are
    interleaved instead: source row i goes to row_start + (i // block) * period +
    i % block (two matrices woven together in groups of `block` rows).  `optional`
    tensors may be absent; when `must_equal` names another parameter, a present
    tensor has to equal it (a tied head stored a second time).

    A rule may take only a part of the stored tensor, and several rules may read the same
    tensor (a checkpoint that stores q, k and v as one matrix, or all experts stacked):
    `source_index` picks [index] of the leading dimension, `transpose` swaps a matrix that is
    stored [in, out], `source_rows` = (first, count) then takes rows of what is left, in that
    order.  `source_shape` is the stored tensor's whole shape; it is needed whenever the part
    taken is not the whole tensor."""

    name: str
    dest: str
    row_start: int = 0
    rows: Optional[int] = None
    optional: bool = False
    must_equal: Optional[str] = None
    block: int = 0
    period: int = 0
    source_shape: Optional[tuple[int, ...]] = None
    source_index: Optional[int] = None
    source_rows: Optional[tuple[int, int]] = None
    transpose: bool = False

    def part_shape(self, stored: tuple[int, ...]) -> tuple[int, ...]:
        """Shape of what this rule takes of a stored tensor of shape `stored`."""
        shape = tuple(stored)
        if self.source_index is not None:
            if not shape or not 0 <= self.source_index < shape[0]:
                raise ValueError(f"weight rule {self.name!r}: source_index {self.source_index} is outside {shape}")
            shape = shape[1:]
        if self.transpose:
            if len(shape) != 2:
                raise ValueError(f"weight rule {self.name!r}: only matrices can be transposed, found {shape}")
            shape = shape[::-1]
        if self.source_rows is not None:
            first, count = self.source_rows
            if not shape or first < 0 or count <= 0 or first + count > shape[0]:
                raise ValueError(f"weight rule {self.name!r}: source_rows {self.source_rows} are outside {shape}")
            shape = (count, *shape[1:])
        return shape

    def take(self, tensor):
        """The part of the stored tensor this rule feeds its destination with."""
        if self.source_index is not None:
            tensor = tensor[self.source_index]
        if self.transpose:
            tensor = tensor.t()
        if self.source_rows is not None:
            first, count = self.source_rows
            tensor = tensor[first : first + count]
        return tensor

    def dest_rows(self, count: int) -> "list[int]":
        """Destination row of each of `count` source rows."""
        if not self.block:
            return list(range(self.row_start, self.row_start + count))
        return [self.row_start + (i // self.block) * self.period + i % self.block for i in range(count)]


@dataclass(frozen=True)
class ModelSpec:
    """Everything `DecoderModel` needs to build a decoder-only model."""

    architecture: str
    vocab_size: int
    hidden_size: int
    max_position_embeddings: int
    layers: tuple[LayerSpec, ...]
    order: tuple[OrderEntry, ...]
    final_norm: PartSpec
    tie_word_embeddings: bool
    weight_rules: tuple[WeightRule, ...]
    init_std: float = 0.02
    # What some decoders do around the layers; the defaults do nothing.
    embedding_scale: float = 1.0  # the embedded tokens times this
    position_embedding: Optional[PartSpec] = None  # a position part whose `embed` is added to the embedded tokens
    head_bias: bool = False  # logits += parameter `head.bias`
    logit_scale: float = 1.0  # logits times this ...
    logit_softcap: Optional[float] = None  # ... then cap * tanh(logits / cap)
