"""Weights from safetensors by tensor name into a model's parameters.

Files: `model.safetensors`, or `model.safetensors.index.json` (a `weight_map`
from tensor name to shard) with its shards; shards without an index are refused
(src/mini_llm_runtime/qwen_loader.py:30-56).  The mapping from names to
parameters is the model spec's `weight_rules`; it is strict both ways, as the
reference's is (src/mini_llm_runtime/qwen_weights.py:55-64, 121-124), but all
problems of a checkpoint are collected into one error.

Element types: matrices take the engine's dtype (bfloat16 or float32); integer
tensors become int32; a vector parameter (norm weight, bias) that the checkpoint
stores in 32-bit stays 32-bit also in the bfloat16 engine.
"""

from __future__ import annotations

import json
from pathlib import Path
from typing import Union

import torch

from ..parts.model import DecoderModel
from ..parts.spec import ParamSpec, WeightRule
from .safetensors_io import SafetensorsFile, TensorEntry


class WeightsError(ValueError):
    """A checkpoint that does not fit the model; lists every missing and unexpected
    tensor and every wrong shape."""

    def __init__(self, missing, unexpected, wrong_shape, other=()):
        self.missing = tuple(missing)
        self.unexpected = tuple(unexpected)
        self.wrong_shape = tuple(wrong_shape)
        self.other = tuple(other)
        lines = ["the checkpoint does not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}):")
            lines += [f"    {n}: found {tuple(f)}, expected {tuple(e)}" for n, f, e in self.wrong_shape]
        lines += [f"  {o}" for o in self.other]
        super().__init__("\n".join(lines))


def checkpoint_files(model_dir: Union[str, Path]) -> dict[str, SafetensorsFile]:
    """Open the checkpoint's files; returns shard name -> file."""
    model_dir = Path(model_dir)
    index = model_dir / "model.safetensors.index.json"
    single = model_dir / "model.safetensors"
    if index.is_file():
        data = json.loads(index.read_text(encoding="utf-8"))
        weight_map = data.get("weight_map") if isinstance(data, dict) else None
        if not isinstance(weight_map, dict) or not weight_map:
            raise ValueError(f"{index} has no weight_map")
        shards = sorted(set(weight_map.values()))
        files = {}
        for shard in shards:
            path = model_dir / shard
            if not path.is_file():
                raise FileNotFoundError(f"{index} names the shard {shard}, which does not exist")
            files[shard] = SafetensorsFile(path)
        problems = []
        for name, shard in weight_map.items():
            if name not in files[shard].entries:
                problems.append(f"index puts {name} into {shard}, which does not hold it")
        listed = set(weight_map)
        for shard, f in files.items():
            for name in f.entries:
                if name not in listed:
                    problems.append(f"{shard} holds {name}, which the index does not list")
        if problems:
            raise ValueError("index and shards disagree: " + "; ".join(problems))
        return files
    if single.is_file():
        return {single.name: SafetensorsFile(single)}
    if any(model_dir.glob("model-*.safetensors")):
        raise FileNotFoundError(f"{model_dir} holds shards but no model.safetensors.index.json")
    raise FileNotFoundError(f"no model.safetensors in {model_dir}")


def _stored_shape(rule: WeightRule, p: ParamSpec) -> tuple[int, ...]:
    """Shape the checkpoint tensor of a rule must have; the part the rule takes of it must be
    what the destination rows want."""
    part = p.shape if rule.rows is None else (rule.rows, *p.shape[1:])
    if rule.source_shape is not None:
        stored = tuple(rule.source_shape)
    elif rule.source_index is not None or rule.source_rows is not None:
        raise ValueError(f"weight rule {rule.name!r} takes a part of its tensor and must give source_shape")
    else:
        stored = tuple(part[::-1]) if rule.transpose else tuple(part)
    if rule.part_shape(stored) != tuple(part):
        raise ValueError(
            f"weight rule {rule.name!r}: it takes {rule.part_shape(stored)} of the stored {stored}, "
            f"{rule.dest} wants {tuple(part)}"
        )
    return stored


def rules_by_tensor(model: DecoderModel) -> dict[str, list[tuple[WeightRule, tuple[int, ...], ParamSpec]]]:
    """Checkpoint tensor name -> the rules that read it, each with the shape the stored tensor
    must have and the parameter it feeds.  Rules that share a tensor must agree on its shape."""
    specs = model.param_specs()
    out: dict[str, list] = {}
    for rule in model.spec.weight_rules:
        if rule.dest not in specs:
            raise KeyError(f"weight rule {rule.name!r} feeds {rule.dest!r}, which the model does not have")
        p = specs[rule.dest]
        shape = _stored_shape(rule, p)
        readers = out.setdefault(rule.name, [])
        if readers:
            if readers[0][1] != shape:
                raise ValueError(f"the rules that read {rule.name!r} expect different shapes: {readers[0][1]} and {shape}")
            if rule.must_equal is not None or readers[0][0].must_equal is not None:
                raise KeyError(f"{rule.name!r}: a tensor that only repeats a parameter cannot feed another")
            if rule.optional != readers[0][0].optional:
                raise KeyError(f"the rules that read {rule.name!r} disagree on whether it may be absent")
        readers.append((rule, shape, p))
    return out


def expected_tensors(model: DecoderModel) -> dict[str, tuple[WeightRule, tuple[int, ...], ParamSpec]]:
    """Checkpoint tensor name -> (its first rule, shape it must have, the parameter that rule feeds)."""
    return {name: readers[0] for name, readers in rules_by_tensor(model).items()}


def _check_coverage(model: DecoderModel) -> None:
    """Every row of every parameter must be fed by exactly one rule."""
    specs = model.param_specs()
    covered: dict[str, list[int]] = {name: [] for name in specs}
    for rule in model.spec.weight_rules:
        if rule.must_equal is not None:
            continue
        rows = specs[rule.dest].shape[0]
        n = rows if rule.rows is None else rule.rows
        covered[rule.dest].extend(rule.dest_rows(n))
    for name, rows in covered.items():
        if sorted(rows) != list(range(specs[name].shape[0])):
            raise ValueError(f"the weight rules do not fill every row of {name} exactly once")


def load_weights(
    model: DecoderModel,
    model_dir: Union[str, Path],
    *,
    dtype: torch.dtype,
    device: Union[str, torch.device],
) -> dict[str, torch.Tensor]:
    """Read the checkpoint into new parameter tensors and bind them to the model."""
    if dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("the engine's dtype is bfloat16 or float32")
    device = torch.device(device)
    _check_coverage(model)
    readers = rules_by_tensor(model)  # rules that do not fit their parameters fail here, before a file is opened
    files = checkpoint_files(model_dir)
    try:
        found: dict[str, TensorEntry] = {}
        duplicates = []
        for shard, f in files.items():
            for name, entry in f.entries.items():
                if name in found:
                    duplicates.append(f"{name} is stored in two files")
                found[name] = entry
        expected = {name: rules[0] for name, rules in readers.items()}
        missing = [n for n, (rule, _, _) in expected.items() if n not in found and not rule.optional]
        unexpected = [n for n in found if n not in expected]
        wrong = [
            (n, found[n].shape, shape) for n, (_, shape, _) in expected.items() if n in found and found[n].shape != shape
        ]
        if missing or unexpected or wrong or duplicates:
            raise WeightsError(missing, unexpected, wrong, duplicates)

        specs = model.param_specs()
        sources: dict[str, list[TensorEntry]] = {name: [] for name in specs}
        for n, rules in readers.items():
            for rule, _, _ in rules:
                if n in found and rule.must_equal is None:
                    sources[rule.dest].append(found[n])
        params: dict[str, torch.Tensor] = {}
        for name, p in specs.items():
            stored = sources[name]
            if stored and all(e.is_integer for e in stored):
                kind = torch.int32
            elif p.keep_stored_precision and stored and all(e.is_32bit_float for e in stored):
                kind = torch.float32
            else:
                kind = dtype
            params[name] = torch.empty(p.shape, dtype=kind, device=device)

        by_file = {f.path: f for f in files.values()}
        checks = []
        for n, rules in readers.items():
            if n not in found:
                continue
            entry = found[n]
            stored = by_file[entry.file].tensor(n)
            for rule, _, _ in rules:
                if rule.must_equal is not None:
                    checks.append((n, rule.must_equal, stored))
                    continue
                tensor = rule.take(stored)
                dest = params[rule.dest]
                rows = dest.shape[0] if rule.rows is None else rule.rows
                if rule.block:
                    index = torch.tensor(rule.dest_rows(rows), dtype=torch.long, device=dest.device)
                    dest.index_copy_(0, index, tensor.to(dest.dtype).to(dest.device))
                else:
                    dest[rule.row_start : rule.row_start + rows].copy_(tensor.to(dest.dtype))
        for n, other, tensor in checks:
            ref = params[other]
            if not torch.equal(tensor.to(ref.dtype).to(ref.device), ref):
                raise WeightsError((), (), (), [f"{n} is stored but differs from {other}, which it must repeat"])
    finally:
        for f in files.values():
            f.close()
    model.bind(params, dtype=dtype, device=device)
    return params
