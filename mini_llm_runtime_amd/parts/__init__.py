"""Parts a layer is put together from, and the model that runs them."""

from . import attention, block, feed_forward, norm, position  # noqa: F401  (register the built-in kinds)
from .base import Block, FeedForward, Mixer, Norm, Part, PositionEncoding
from .context import KVView, StateView, StepContext
from .model import DecoderModel
from .registry import build_part, part_kinds, register_part, unregister_part
from .spec import LayerSpec, ModelSpec, OrderEntry, ParamSpec, PartSpec, WeightRule

__all__ = [
    "Block",
    "DecoderModel",
    "FeedForward",
    "KVView",
    "LayerSpec",
    "Mixer",
    "ModelSpec",
    "Norm",
    "OrderEntry",
    "ParamSpec",
    "Part",
    "PartSpec",
    "PositionEncoding",
    "StateView",
    "StepContext",
    "WeightRule",
    "build_part",
    "part_kinds",
    "register_part",
    "unregister_part",
]
