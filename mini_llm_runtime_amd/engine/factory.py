"""Putting the pieces together: a model folder becomes a model, a cache manager
and a runner.  The reference does the same wiring by hand in its scripts
(experiments/continuous_batch_engine_runner.py:227-254)."""

from __future__ import annotations

from pathlib import Path
from typing import Any, Optional, Sequence, Union

import torch

from ..cache.manager import CacheManager
from ..config.model_config import ModelConfig
from ..models.registry import build_model, load_config
from ..parts.model import DecoderModel
from ..weights.loader import load_weights

DTYPES = {
    "bfloat16": torch.bfloat16,
    "bf16": torch.bfloat16,
    "float32": torch.float32,
    "fp32": torch.float32,
}


def parse_dtype(name: Union[str, torch.dtype]) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError("the engine's dtype is bfloat16 or float32")
        return name
    try:
        return DTYPES[name]
    except KeyError:
        raise ValueError(f"unknown dtype {name!r}; use bfloat16 or float32") from None


def default_ops(dtype: torch.dtype, device: Union[str, torch.device]) -> Any:
    """The HIP kernel library; raises when it cannot be built or there is no GPU."""
    from ..kernels.ops import HipOps

    return HipOps(dtype=dtype, device=device)


def load_model(
    model_dir: Union[str, Path],
    *,
    dtype: Union[str, torch.dtype] = "bfloat16",
    device: Union[str, torch.device] = "cuda",
) -> tuple[ModelConfig, DecoderModel]:
    """config.json chooses the model class; weights come from the safetensors beside it."""
    dtype = parse_dtype(dtype)
    config = load_config(model_dir)
    model = build_model(config)
    load_weights(model, model_dir, dtype=dtype, device=device)
    return config, model


def make_cache(
    model: DecoderModel,
    *,
    block_size: int,
    num_blocks: Union[int, Sequence[int]],
    max_requests: int,
    dtype: Optional[torch.dtype] = None,
    device: Optional[Union[str, torch.device]] = None,
) -> CacheManager:
    return CacheManager(
        model.site_cache_specs(),
        block_size=block_size,
        num_blocks=num_blocks,
        max_requests=max_requests,
        dtype=dtype or model.dtype,
        device=device or model.device,
    )
