"""Drawn configurations of the architecture through the step function: head counts and groups, head
sizes in steps of 16, widths that are no multiple of 8 (the products then take the kernels without
matrix cores), intermediate sizes and vocabularies of any even and any size, page sizes from 4 to 32:
each under a drawn schedule (mixed requests with pages used again, portions, bulk and tail) and dtype,
against the plain implementation."""

from __future__ import annotations

import random

import pytest
import torch

import helpers
import schedules
import test_step_schedules as families
from helpers import random_tokens

pytestmark = pytest.mark.gpu


def _draw(case: int):
    rng = random.Random(5000 + case)
    kv = rng.choice([1, 1, 2, 3, 4])
    heads = kv * rng.choice([1, 2, 3, 4, 7, 8])
    d = rng.choice([16, 32, 48, 64, 80, 96, 128])
    hidden = rng.choice([8 * rng.randint(3, 70), 8 * rng.randint(3, 70), 4 * rng.randint(7, 60) + 2,
                         heads * d if heads * d <= 640 else 8 * rng.randint(3, 70)])
    inter = rng.choice([4 * rng.randint(5, 150), 2 * rng.randint(9, 200), 2 * rng.randint(9, 100)])
    config = dict(
        architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=rng.randint(40, 700), hidden_size=hidden,
        intermediate_size=inter, num_hidden_layers=rng.randint(1, 3), num_attention_heads=heads, num_key_value_heads=kv,
        head_dim=d, max_position_embeddings=512, rms_norm_eps=rng.choice([1e-5, 1e-6]), rope_theta=rng.choice([1e4, 1e6]),
        hidden_act="silu", tie_word_embeddings=rng.random() < 0.5,
    )
    block_size = rng.choice([4, 8, 16, 32])
    dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float32])
    lengths = [rng.choice([1, 2, 3, rng.randint(4, 40), rng.randint(30, 140), rng.randint(100, 300)])
               for _ in range(rng.randint(3, 6))]
    family = rng.choice(["mixed", "mixed", "portions", "bulk_then_tail"])
    return config, block_size, dtype, lengths, family


@pytest.mark.parametrize("case", range(60, 84))
def test_a_drawn_configuration_under_a_drawn_schedule(tmp_path, case):
    config, block_size, dtype, lengths, family = _draw(case)
    name = f"drawn{case}"
    helpers.TINY[name], helpers.BLOCK_SIZE[name] = config, block_size
    try:
        requests = {f"r{i}": random_tokens(n, config["vocab_size"], 9000 + 13 * case + i) for i, n in enumerate(lengths)}
        steps = schedules.mixed(requests, seed=case) if family == "mixed" else families.FAMILIES[family](requests)
        cfg, weights, cache, runner = families._setup(tmp_path, name, "hip", dtype, steps)
        got = schedules.run_schedule(runner, cache, steps)
        families._compare(got, requests, weights, cfg, dtype, row_bound=0.12)
        cache.check_invariants()
    finally:
        del helpers.TINY[name], helpers.BLOCK_SIZE[name]
