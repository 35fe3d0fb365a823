"""One request through the step function by itself: its prompt in one step, then a token per step.

The entry point and what it reports have the reference's names
(src/mini_llm_runtime/generation.py:29-117): N new tokens cost one prompt step and at most
N - 1 decode steps; the last generated token is never fed back, so the cache ends at
prompt + N - 1 tokens (generation.py:41-42); room in the cache is checked before anything is
written (generation.py:53-57, 74-80); a stop token ends the run without a further step.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Collection, Iterator, Optional, Sequence, Union

import torch

from ..sampling.sampler import GREEDY, Sampler, SamplingParams
from .runner import ModelRunner, StepEntry


@dataclass(frozen=True)
class GenerationOutput:
    generated_token_ids: tuple[int, ...]
    stopped_by_eos: bool
    prefill_tokens: int
    decode_steps: int
    cache_length: int
    step_logits: Optional[tuple[torch.Tensor, ...]] = None


def _stop_set(eos_token_ids: Union[int, Collection[int], None], vocab_size: int) -> frozenset[int]:
    if eos_token_ids is None:
        return frozenset()
    stops = frozenset([eos_token_ids] if isinstance(eos_token_ids, int) else (int(t) for t in eos_token_ids))
    outside = sorted(t for t in stops if not 0 <= t < vocab_size)
    if outside:
        raise ValueError(f"EOS token ids outside the vocabulary: {outside}")
    return stops


def _token_stream(
    runner: ModelRunner, sampler: Sampler, request_id: str, prompt: Sequence[int], sampling: SamplingParams, limit: int
) -> Iterator[tuple[int, torch.Tensor]]:
    """(token, the logits it was chosen from) for up to `limit` tokens; every `next` runs one
    step: the prompt first, then the token chosen last."""
    feed = list(prompt)
    for index in range(limit):
        out = runner.step([StepEntry.of(request_id, feed, (len(feed) - 1,))], borrow_logits=True)
        token = int(sampler.sample(out.logits, [sampling], [index]).cpu()[0])
        yield token, out.logits[0]
        feed = [token]


@torch.inference_mode()
def generate(
    runner: ModelRunner,
    input_ids: Sequence[int],
    *,
    max_new_tokens: int,
    eos_token_ids: Union[int, Collection[int], None] = None,
    sampling: SamplingParams = GREEDY,
    return_step_logits: bool = False,
    request_id: str = "generate",
) -> GenerationOutput:
    prompt = [int(t) for t in input_ids]
    if not prompt:
        raise ValueError("the prompt must not be empty")
    if max_new_tokens <= 0:
        raise ValueError("max_new_tokens must be > 0")
    most_cached = len(prompt) + max_new_tokens - 1
    if most_cached > runner.max_positions:
        raise ValueError("prompt length + max_new_tokens - 1 exceeds max_position_embeddings")
    stops = _stop_set(eos_token_ids, runner.vocab_size)
    cache = runner.cache
    for group in cache.groups:
        need = group.lifetime_blocks(most_cached, len(prompt))
        if need > group.allocator.available_count:
            raise RuntimeError(
                f"the cache has {group.allocator.available_count} free pages in group {group.index}, "
                f"generation needs {need}"
            )
    tokens: list[int] = []
    kept: list[torch.Tensor] = []
    stopped = False
    cache.create_request(request_id)
    try:
        stream = _token_stream(runner, Sampler(runner.ops, runner.device), request_id, prompt, sampling, max_new_tokens)
        for token, logits in stream:
            tokens.append(token)
            if return_step_logits:
                kept.append(logits.clone())  # the step's buffer may be a recording's own
            if token in stops:
                stopped = True
                break  # before the stream feeds it back: no step is spent on a stop token
        cached = cache.get_request(request_id).num_tokens
    finally:
        cache.release_request(request_id)
    return GenerationOutput(
        generated_token_ids=tuple(tokens),
        stopped_by_eos=stopped,
        prefill_tokens=len(prompt),
        decode_steps=len(tokens) - 1,
        cache_length=cached,
        step_logits=tuple(kept) if return_step_logits else None,
    )


def greedy_generate(
    runner: ModelRunner,
    input_ids: Sequence[int],
    *,
    max_new_tokens: int,
    eos_token_ids: Union[int, Collection[int], None] = None,
    return_step_logits: bool = False,
) -> GenerationOutput:
    """Greedy generation; name and arguments as the reference's entry point."""
    return generate(
        runner,
        input_ids,
        max_new_tokens=max_new_tokens,
        eos_token_ids=eos_token_ids,
        sampling=GREEDY,
        return_step_logits=return_step_logits,
    )


__all__ = ["GenerationOutput", "generate", "greedy_generate"]
