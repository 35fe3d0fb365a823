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

from .config import blocks_for_memory, parse_dtype  # noqa: F401  (parse_dtype is part of this module's surface)


def default_ops(dtype: torch.dtype, device: Union[str, torch.device], tuning: Any = None) -> Any:
    """The HIP kernel library; raises when it cannot be built or there is no GPU."""
    from ..kernels.ops import HipOps

    return HipOps(dtype=dtype, device=device, tuning=tuning)


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
    check_visibility: bool = False,
) -> CacheManager:
    return CacheManager(
        model.site_cache_specs(),
        block_size=block_size,
        num_blocks=num_blocks,
        max_requests=max_requests,
        dtype=dtype or model.dtype,
        device=device or model.device,
        check_visibility=check_visibility,
    )


def page_bytes(model: DecoderModel, block_size: int, dtype: torch.dtype) -> int:
    """Bytes one page id costs over all page pools of a model (every pool is given the same
    number of pages): keys and values of every site that owns pages."""
    width = torch.empty((), dtype=dtype).element_size()
    total = 0
    for spec in model.site_cache_specs():
        if spec is not None:
            total += spec.page_bytes(block_size, width)  # 0 for what does not live in pages
    return total


def recording_reserve_bytes(
    model: DecoderModel, limits: Any, dtype: torch.dtype, max_running_requests: int, max_batch_tokens: int
) -> int:
    """An upper estimate of what the step function's recorded steps hold beside the weights and the
    page pool: every recording owns its activations (per token about twice the output widths of one
    layer's matrices, for tensors that live side by side, plus two float32 copies of the stream) and a
    float32 logits buffer [wanted rows, vocab].  Single-token recordings exist per (batch padded to a
    power of two, block table width), other steps per shape; `limits` (a `GraphLimits`) bounds both."""
    if limits is None or not limits.enabled:
        return 0
    width = torch.empty((), dtype=dtype).element_size()
    spec = model.spec
    layer_widths = 0
    for name, p in model.param_specs().items():
        if name.startswith("layers.0.") and len(p.shape) == 2:
            layer_widths += int(p.shape[0])
    per_token = 2 * layer_widths * width + 8 * spec.hidden_size
    logits_row = spec.vocab_size * 4
    largest = 1
    while largest < min(max_running_requests, limits.max_decode_batch):
        largest *= 2
    batches = []
    b = 1
    while b <= largest:
        batches.append(b)
        b *= 2
    widths_each = -(-limits.max_decode_graphs // len(batches))
    decode = sum(b * (per_token + logits_row) for b in batches) * widths_each
    step_tokens = min(limits.max_step_tokens, max_batch_tokens)
    steps = limits.max_step_graphs * (step_tokens * per_token + max_running_requests * logits_row)
    return decode + steps


def blocks_from_free_memory(
    model: DecoderModel,
    block_size: int,
    dtype: torch.dtype,
    device: torch.device,
    fraction: float,
    reserve_bytes: int = 0,
) -> int:
    """Pages per pool that `fraction` of the device memory free right now holds, after
    `reserve_bytes` were set aside (for recorded steps: at most half of what is free)."""
    per_page = page_bytes(model, block_size, dtype)
    if per_page == 0:
        return 1  # a model without paged sites still gets a (never used) pool
    if device.type != "cuda":
        raise ValueError("kv_memory_fraction needs a GPU; give num_blocks instead")
    free, _ = torch.cuda.mem_get_info(device)
    free -= min(int(reserve_bytes), free // 2)
    return blocks_for_memory(per_page, free, fraction)
