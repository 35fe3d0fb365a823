"""Tiny configurations and small utilities shared by the tests."""

from __future__ import annotations

import json
from pathlib import Path

import torch

from mini_llm_runtime_amd.config import Qwen2Config
from mini_llm_runtime_amd.config.presets import load_preset
from mini_llm_runtime_amd.engine.factory import load_model, make_cache
from mini_llm_runtime_amd.engine.runner import ModelRunner, StepEntry
from mini_llm_runtime_amd.weights import SafetensorsFile, write_random_model

# Two tiny Qwen2 configurations that differ in every size and option.
TINY_A = dict(
    architectures=["Qwen2ForCausalLM"],
    model_type="qwen2",
    vocab_size=256,
    hidden_size=64,
    intermediate_size=128,
    num_hidden_layers=2,
    num_attention_heads=4,
    num_key_value_heads=2,
    max_position_embeddings=512,
    rms_norm_eps=1e-6,
    rope_theta=10000.0,
    hidden_act="silu",
    tie_word_embeddings=True,
)
TINY_B = dict(
    architectures=["Qwen2ForCausalLM"],
    model_type="qwen2",
    vocab_size=517,
    hidden_size=96,
    intermediate_size=352,
    num_hidden_layers=3,
    num_attention_heads=3,
    num_key_value_heads=1,
    head_dim=32,
    max_position_embeddings=1024,
    rms_norm_eps=1e-5,
    rope_theta=1000000.0,
    hidden_act="silu",
    tie_word_embeddings=False,
)
# Two more, with sizes that kernels dislike.  C: a head size that is not hidden / heads, a
# group of three, one layer, an odd vocabulary.  D: a width and a feed-forward width that are
# no multiples of 8 and a head size that is no multiple of 16 (the matrix-core kernels refuse
# them and the plain 32-bit kernels take over), as many key/value heads as query heads.
TINY_C = dict(
    architectures=["Qwen2ForCausalLM"],
    model_type="qwen2",
    vocab_size=1003,
    hidden_size=72,
    intermediate_size=200,
    num_hidden_layers=1,
    num_attention_heads=6,
    num_key_value_heads=2,
    head_dim=48,
    max_position_embeddings=256,
    rms_norm_eps=3e-6,
    rope_theta=500000.0,
    hidden_act="silu",
    tie_word_embeddings=True,
)
TINY_D = dict(
    architectures=["Qwen2ForCausalLM"],
    model_type="qwen2",
    vocab_size=300,
    hidden_size=100,
    intermediate_size=108,
    num_hidden_layers=2,
    num_attention_heads=5,
    num_key_value_heads=5,
    max_position_embeddings=300,
    rms_norm_eps=1e-4,
    rope_theta=777.0,
    hidden_act="silu",
    tie_word_embeddings=False,
)
# E: the `tiny-b` preset as it ships (width 128, four query heads on ONE key/value head: a group
# of four; vocabulary 512, untied head), which the entry points' smoke run and the command line use.
TINY_E = {k: v for k, v in load_preset("tiny-b").items() if k not in ("torch_dtype", "use_sliding_window")}
TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E}
BLOCK_SIZE = {"A": 16, "B": 8, "C": 32, "D": 4, "E": 8}


def make_model_dir(tmp_path: Path, which: str, seed: int = 0, storage_dtype: str = "bfloat16") -> Path:
    config = Qwen2Config.from_dict(TINY[which])
    return write_random_model(config, Path(tmp_path) / f"tiny{which}", seed=seed, storage_dtype=storage_dtype)


def read_weights(model_dir: Path) -> tuple[dict, dict[str, torch.Tensor]]:
    """(config dict, checkpoint tensors) for the plain implementation."""
    cfg = json.loads((Path(model_dir) / "config.json").read_text())
    with SafetensorsFile(Path(model_dir) / "model.safetensors") as f:
        tensors = {name: f.tensor(name) for name in f.entries}
    return cfg, tensors


def make_runner(model_dir: Path, ops, *, block_size: int, num_blocks: int, max_requests: int = 8):
    config, model = load_model(model_dir, dtype=ops.dtype, device=ops.device)
    cache = make_cache(model, block_size=block_size, num_blocks=num_blocks, max_requests=max_requests)
    return config, model, cache, ModelRunner(model, cache, ops)


def random_tokens(count: int, vocab: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (count,), generator=g).tolist()


__all__ = [
    "BLOCK_SIZE",
    "StepEntry",
    "TINY",
    "TINY_A",
    "TINY_B",
    "make_model_dir",
    "make_runner",
    "random_tokens",
    "read_weights",
]
