"""Single-request generation over the step function: one whole-prompt step, then
one token per step.

Same control loop and counts as the reference's `greedy_generate`
(src/mini_llm_runtime/generation.py:29-117): N new tokens cost one prompt step and
at most N-1 decode steps; the last generated token is never fed back, so the cache
ends at prompt + N - 1 tokens (generation.py:41-42); capacity is checked before
anything is written (generation.py:53-57, 74-80); EOS stops without a further step.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Collection, Optional, Sequence, Union

import torch

from ..cache.block_pool import blocks_for
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


def _normalize_eos(eos_token_ids: Union[int, Collection[int], None], vocab_size: int) -> frozenset[int]:
    if eos_token_ids is None:
        return frozenset()
    values = {eos_token_ids} if isinstance(eos_token_ids, int) else {int(t) for t in eos_token_ids}
    invalid = sorted(t for t in values if not 0 <= t < vocab_size)
    if invalid:
        raise ValueError(f"EOS token ids outside the vocabulary: {invalid}")
    return frozenset(values)


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
    required = len(prompt) + max_new_tokens - 1
    if required > runner.max_positions:
        raise ValueError("prompt length + max_new_tokens - 1 exceeds max_position_embeddings")
    eos = _normalize_eos(eos_token_ids, runner.vocab_size)
    cache = runner.cache
    for group in cache.groups:
        need = group.lifetime_blocks(required, len(prompt))
        if need > group.allocator.available_count:
            raise RuntimeError(
                f"the cache has {group.allocator.available_count} free pages in group {group.index}, "
                f"generation needs {need}"
            )
    sampler = Sampler(runner.ops, runner.device)
    cache.create_request(request_id)
    generated: list[int] = []
    captured: Optional[list[torch.Tensor]] = [] if return_step_logits else None
    stopped = False
    decode_steps = 0
    try:
        tokens = prompt
        for index in range(max_new_tokens):
            out = runner.step([StepEntry.of(request_id, tokens, (len(tokens) - 1,))], borrow_logits=True)
            if captured is not None:
                captured.append(out.logits[0].clone())
            nxt = int(sampler.sample(out.logits, [sampling], [index]).cpu()[0])
            generated.append(nxt)
            if index > 0:
                decode_steps += 1
            stopped = nxt in eos
            if stopped or index == max_new_tokens - 1:
                break
            tokens = [nxt]
        cache_length = cache.get_request(request_id).num_tokens
    finally:
        cache.release_request(request_id)
    return GenerationOutput(
        generated_token_ids=tuple(generated),
        stopped_by_eos=stopped,
        prefill_tokens=len(prompt),
        decode_steps=decode_steps,
        cache_length=cache_length,
        step_logits=tuple(captured) if captured is not None else None,
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


__all__ = ["GenerationOutput", "generate", "greedy_generate", "blocks_for"]
