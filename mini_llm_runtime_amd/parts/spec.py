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
    tensor has to equal it (a tied head stored a second time)."""

    name: str
    dest: str
    row_start: int = 0
    rows: Optional[int] = None
    optional: bool = False
    must_equal: Optional[str] = None
    block: int = 0
    period: int = 0

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
