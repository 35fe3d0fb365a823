"""Choosing the next token from logits: greedy, or temperature sampling.

The reference chooses greedily only (`argmax` on the GPU, src/mini_llm_runtime/engine.py:222,
246; generation.py:95).  Temperature sampling is added here: p = softmax(logits /
temperature) in 32-bit, and the token is the first whose cumulative probability
exceeds a uniform number.  That number comes from a counter-based generator keyed by
the request's seed and the index of the token being generated, so a request's
sampled tokens do not depend on what else is in the batch or on how its prompt was
cut into steps.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Sequence

import numpy as np
import torch


@dataclass(frozen=True)
class SamplingParams:
    """temperature 0 means greedy.  `seed` keys the request's random numbers."""

    temperature: float = 0.0
    seed: int = 0

    def __post_init__(self) -> None:
        if not self.temperature >= 0.0:
            raise ValueError("temperature must be >= 0")
        if isinstance(self.seed, bool) or not isinstance(self.seed, int) or self.seed < 0:
            raise ValueError("seed must be a non-negative integer")


GREEDY = SamplingParams()


def uniform_for(seed: int, token_index: int) -> float:
    """The uniform number in [0, 1) for the `token_index`-th generated token of a request."""
    key = np.array([seed & 0xFFFFFFFFFFFFFFFF, (seed >> 64) & 0xFFFFFFFFFFFFFFFF], dtype=np.uint64)
    counter = np.array([token_index, 0, 0, 0], dtype=np.uint64)
    bits = np.random.Philox(key=key, counter=counter).random_raw(1)[0]
    # 24 bits: exactly representable in float32 and never 1.0
    return float(int(bits) >> 40) / float(1 << 24)


class Sampler:
    def __init__(self, ops: Any, device: torch.device) -> None:
        self.ops = ops
        self.device = torch.device(device)

    def sample(
        self,
        logits: torch.Tensor,
        params: Sequence[SamplingParams],
        token_indices: Sequence[int],
    ) -> torch.Tensor:
        """int32 [K] on the device: one token per logits row."""
        if logits.shape[0] != len(params) or len(params) != len(token_indices):
            raise ValueError("one SamplingParams and one token index per logits row")
        if all(p.temperature == 0.0 for p in params):
            return self.ops.sample(logits, None, None)
        host = np.empty((2, len(params)), dtype=np.float32)
        for i, (p, n) in enumerate(zip(params, token_indices)):
            host[0, i] = p.temperature
            host[1, i] = uniform_for(p.seed, n) if p.temperature > 0 else 0.0
        dev = torch.from_numpy(host).to(self.device)
        return self.ops.sample(logits, dev[0], dev[1])
