"""Random-weights mode: write a model folder (config.json, model.safetensors) from
a configuration and a seed.

Every tensor is drawn from a generator seeded by the seed and the tensor's own
name, so the result does not depend on the order in which tensors are made:
matrices and biases ~ N(0, std), norm weights 1 + N(0, std)  (std from the model
spec, 0.02).  The reference has random weights only in its tests
(tests/test_qwen_weights.py:25-65, `torch.randn` with seed 7).
"""

from __future__ import annotations

import json
import zlib
from pathlib import Path
from typing import Iterator, Union

import torch

from ..config.model_config import ModelConfig
from ..parts.model import DecoderModel
from ..parts.spec import ParamSpec
from .loader import expected_tensors
from .safetensors_io import write_safetensors

_STORAGE = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def _generator(seed: int, name: str) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed((int(seed) * 1_000_003 + zlib.crc32(name.encode("utf-8"))) % (2**63 - 1))
    return g


def random_tensor(name: str, shape: tuple[int, ...], spec: ParamSpec, seed: int, std: float, dtype: torch.dtype) -> torch.Tensor:
    values = torch.randn(shape, generator=_generator(seed, name), dtype=torch.float32) * std
    if spec.init == "one_plus_normal":
        values += 1.0
    elif spec.init != "normal":
        raise ValueError(f"unknown init {spec.init!r} for {name}")
    return values.to(dtype)


def random_checkpoint_tensors(
    model: DecoderModel, seed: int, dtype: torch.dtype
) -> tuple[list[tuple[str, torch.dtype, tuple[int, ...]]], Iterator[tuple[str, torch.Tensor]]]:
    """(layout, stream) of the checkpoint tensors a model expects, in rule order."""
    std = model.spec.init_std
    wanted = [
        (name, shape, p)
        for name, (rule, shape, p) in expected_tensors(model).items()
        if rule.must_equal is None
    ]
    layout = [(name, dtype, shape) for name, shape, _ in wanted]

    def stream() -> Iterator[tuple[str, torch.Tensor]]:
        for name, shape, p in wanted:
            yield name, random_tensor(name, shape, p, seed, std, dtype)

    return layout, stream()


def write_random_model(
    config: ModelConfig,
    folder: Union[str, Path],
    *,
    seed: int = 0,
    storage_dtype: str = "bfloat16",
) -> Path:
    """Write `<folder>/config.json` and `<folder>/model.safetensors`; returns the folder."""
    from ..models.registry import build_model

    if storage_dtype not in _STORAGE:
        raise ValueError(f"storage_dtype must be one of {sorted(_STORAGE)}")
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    model = build_model(config)
    path = config.save(folder)
    # the stored element type, under the key checkpoints carry it in: an engine that is not told a
    # dtype computes in this one
    data = json.loads(path.read_text(encoding="utf-8"))
    data["torch_dtype"] = storage_dtype
    path.write_text(json.dumps(data, indent=2) + "\n", encoding="utf-8")
    layout, stream = random_checkpoint_tensors(model, seed, _STORAGE[storage_dtype])
    write_safetensors(
        folder / "model.safetensors",
        layout,
        stream,
        metadata={"format": "pt", "seed": str(int(seed)), "source": "random weights"},
    )
    return folder


def bind_random_weights(
    model: DecoderModel,
    *,
    seed: int,
    dtype: torch.dtype,
    device: Union[str, torch.device],
) -> dict[str, torch.Tensor]:
    """Random parameters made on the device, one tensor at a time, and bound to the model:
    the same distributions as the folder mode (matrices and biases ~ N(0, std), norm weights
    1 + N(0, std)) without the trip through a file, so that a 64 GB model is there in seconds.
    Every tensor's generator is seeded by the seed and the parameter's name.  The values are
    not those of `write_random_model` (another generator, and parameters instead of checkpoint
    tensors), so a comparison with a plain implementation takes the folder mode."""
    device = torch.device(device)
    std = model.spec.init_std
    params: dict[str, torch.Tensor] = {}
    for name, spec in model.param_specs().items():
        g = torch.Generator(device=device)
        g.manual_seed((int(seed) * 1_000_003 + zlib.crc32(name.encode("utf-8"))) % (2**63 - 1))
        kind = torch.float32 if spec.keep_stored_precision else dtype
        t = torch.empty(spec.shape, dtype=kind, device=device)
        t.normal_(0.0, std, generator=g)
        if spec.init == "one_plus_normal":
            t += 1.0
        elif spec.init != "normal":
            raise ValueError(f"unknown init {spec.init!r} for {name}")
        params[name] = t
    model.bind(params, dtype=dtype, device=device)
    return params
