"""Everything an engine is set up with, in one typed object.

The reference wires these values by hand where it builds an engine
(experiments/continuous_batch_engine_runner.py:233-254: dtype, total_blocks,
block_size, max_running_requests, max_batch_tokens); here they are one dataclass that
`ContinuousBatchEngine.from_model_dir` and the command line consume.  Nothing in it
is a property of the model: sizes of the model come from its config.json.
"""

from __future__ import annotations

from dataclasses import dataclass, fields, replace
from typing import Any, Mapping, Optional, Union

import torch

from ..kernels.tuning import KernelTuning
from .scheduler import BatchingPolicy

_DTYPE_NAMES = {
    "bfloat16": torch.bfloat16,
    "bf16": torch.bfloat16,
    "float32": torch.float32,
    "fp32": torch.float32,
    "float": torch.float32,
}


def parse_dtype(name: Union[str, torch.dtype]) -> torch.dtype:
    """The engine computes in bfloat16 or in true float32."""
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError("the engine's dtype is bfloat16 or float32")
        return name
    try:
        return _DTYPE_NAMES[name]
    except KeyError:
        raise ValueError(f"unknown dtype {name!r}; use bfloat16 or float32") from None


def dtype_of_checkpoint(config_json: Mapping[str, Any]) -> torch.dtype:
    """The dtype a model folder asks for: config.json's `torch_dtype` when it names one the
    engine computes in; float16 checkpoints run in bfloat16 (same width, the engine has no
    float16 path); anything else, or no key, runs in bfloat16."""
    stored = config_json.get("torch_dtype")
    if stored in ("float32", "fp32"):
        return torch.float32
    return torch.bfloat16


@dataclass(frozen=True)
class GraphLimits:
    """How many recorded steps the step function keeps, and how large they may be.  A
    recording owns its activations and a [wanted rows, vocab] float32 logits buffer
    (for 256 rows of a 152k vocabulary: 155 MB), so the limits bound device memory that
    the page pool does not see."""

    enabled: bool = True
    max_decode_graphs: int = 64  # (padded batch, table width) shapes of single-token steps
    max_decode_batch: int = 256  # larger single-token batches run unrecorded
    max_step_graphs: int = 16  # shapes of other steps (prompt portions, mixed batches)
    max_step_tokens: int = 8192  # larger steps run unrecorded

    def __post_init__(self) -> None:
        for f in fields(self):
            value = getattr(self, f.name)
            if f.name != "enabled" and (isinstance(value, bool) or not isinstance(value, int) or value <= 0):
                raise ValueError(f"GraphLimits.{f.name} must be a positive integer")


@dataclass(frozen=True)
class EngineConfig:
    """dtype: None takes config.json's `torch_dtype` (see `dtype_of_checkpoint`).
    The page pool is sized by `num_blocks`, or, when that is None, by
    `kv_memory_fraction` of the device memory that is free once the weights are loaded."""

    dtype: Optional[Union[str, torch.dtype]] = None
    device: Union[str, torch.device] = "cuda"
    block_size: int = 16
    num_blocks: Optional[int] = None
    kv_memory_fraction: float = 0.8
    max_running_requests: int = 8
    max_batch_tokens: int = 2048
    max_mixed_prefill_tokens: Optional[int] = None
    batching_policy: BatchingPolicy = BatchingPolicy.CONTINUOUS
    lookahead: bool = True
    enable_tracing: bool = False
    check_cache_visibility: bool = False  # debug: refuse reads of a site's pending tokens before its write
    graphs: GraphLimits = GraphLimits()
    tuning: KernelTuning = KernelTuning()

    def __post_init__(self) -> None:
        if self.dtype is not None:
            parse_dtype(self.dtype)
        for name in ("block_size", "max_running_requests", "max_batch_tokens"):
            value = getattr(self, name)
            if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
                raise ValueError(f"EngineConfig.{name} must be a positive integer")
        if self.num_blocks is not None and (not isinstance(self.num_blocks, int) or self.num_blocks <= 0):
            raise ValueError("EngineConfig.num_blocks must be a positive integer or None")
        if not 0.0 < float(self.kv_memory_fraction) <= 1.0:
            raise ValueError("EngineConfig.kv_memory_fraction must lie in (0, 1]")
        if not isinstance(self.batching_policy, BatchingPolicy):
            raise ValueError("EngineConfig.batching_policy must be a BatchingPolicy")

    def with_overrides(self, **changes: Any) -> "EngineConfig":
        """A copy with some fields replaced; unknown names are an error."""
        known = {f.name for f in fields(self)}
        unknown = sorted(set(changes) - known)
        if unknown:
            raise TypeError(f"EngineConfig has no field {', '.join(unknown)}")
        return replace(self, **changes)

    def resolved_dtype(self, config_json: Mapping[str, Any]) -> torch.dtype:
        return parse_dtype(self.dtype) if self.dtype is not None else dtype_of_checkpoint(config_json)


def blocks_for_memory(bytes_per_block: int, free_bytes: int, fraction: float) -> int:
    """Pages that `fraction` of `free_bytes` holds."""
    if bytes_per_block <= 0:
        raise ValueError("bytes_per_block must be > 0")
    count = int(free_bytes * fraction) // bytes_per_block
    if count <= 0:
        raise ValueError(
            f"{fraction:.2f} of {free_bytes} free bytes hold no page of {bytes_per_block} bytes"
        )
    return count
