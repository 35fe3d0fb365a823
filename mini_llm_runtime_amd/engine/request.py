"""One request as the engine sees it: its prompt, how much of it is in the cache, the tokens
it has produced, why it ended, and when things happened to it.

The reference spreads this over three structures that are kept in step by hand: the
scheduler's request record (src/mini_llm_runtime/scheduler.py:34-70), the metrics collector's
timeline (request_metrics.py:97-116) and the engine's bookkeeping between them.  Here it is
one object that the scheduler moves between its queues, the engine stamps, and the figures
(time to first token, time between tokens, ...) are read from.
"""

from __future__ import annotations

import statistics
from dataclasses import dataclass, field
from enum import Enum
from typing import Optional, Sequence

from ..sampling.sampler import GREEDY, SamplingParams


class Phase(str, Enum):
    QUEUED = "queued"  # submitted, not yet admitted
    ACTIVE = "active"  # admitted: its prompt is being consumed or it decodes
    DONE = "done"


class EndReason(str, Enum):
    STOP_TOKEN = "eos"
    LENGTH = "max_tokens"


def _ms(ns) -> Optional[float]:
    return None if ns is None else ns / 1e6


@dataclass
class Timeline:
    """Moments of a request's life on one monotonic clock, in nanoseconds.  A token's moment
    is when the host can see it (after the copy from the device); everything counts from the
    arrival, and the end-to-end time ends at the last token: what the engine does afterwards
    (giving pages back) is `cleanup` (definitions of request_metrics.py:20-94 of the reference)."""

    arrived: Optional[int] = None
    scheduled: list[int] = field(default_factory=list)  # the prompt's first portion entered a step (again after a failed one)
    tokens: list[int] = field(default_factory=list)
    done: Optional[int] = None

    def _latest(self) -> int:
        moments = [m for m in (self.arrived, self.done) if m is not None] + self.scheduled + self.tokens
        return max(moments, default=0)

    def stamp(self, what: str, moment: int) -> None:
        if isinstance(moment, bool) or not isinstance(moment, int) or moment < 0:
            raise ValueError("a moment is a non-negative integer of nanoseconds")
        if moment < self._latest():
            raise ValueError("a request's moments must not go back in time")
        if what == "arrived":
            if self.arrived is not None:
                raise RuntimeError("the request has arrived already")
            self.arrived = moment
        elif self.arrived is None:
            raise RuntimeError("nothing happens to a request before it arrives")
        elif self.done is not None:
            raise RuntimeError("nothing happens to a request after it is done")
        elif what == "scheduled":
            if self.tokens:
                raise RuntimeError("a request that produced tokens does not start its prompt again")
            self.scheduled.append(moment)
        elif what == "token":
            self.tokens.append(moment)
        elif what == "done":
            if not self.tokens:
                raise RuntimeError("a request without tokens cannot be done")
            self.done = moment
        else:
            raise ValueError(f"unknown moment {what!r}")

    # ---- figures, in nanoseconds (None while they cannot be known) -----------------------------
    @property
    def queue_wait_ns(self) -> Optional[int]:
        return self.scheduled[0] - self.arrived if self.scheduled else None

    @property
    def ttft_ns(self) -> Optional[int]:
        return self.tokens[0] - self.arrived if self.tokens else None

    @property
    def gaps_ns(self) -> tuple[int, ...]:
        return tuple(b - a for a, b in zip(self.tokens, self.tokens[1:]))

    @property
    def median_gap_ns(self) -> Optional[float]:
        gaps = self.gaps_ns
        return float(statistics.median(gaps)) if gaps else None

    @property
    def e2e_ns(self) -> Optional[int]:
        return self.tokens[-1] - self.arrived if self.tokens else None

    @property
    def cleanup_ns(self) -> Optional[int]:
        return self.done - self.tokens[-1] if self.done is not None and self.tokens else None

    def figures_ms(self) -> dict[str, Optional[float]]:
        """queue wait, time to first token, median time between tokens, end to end, clean-up."""
        return {
            "queue_wait_ms": _ms(self.queue_wait_ns),
            "ttft_ms": _ms(self.ttft_ns),
            "median_tpot_ms": _ms(self.median_gap_ns),
            "e2e_ms": _ms(self.e2e_ns),
            "cleanup_ms": _ms(self.cleanup_ns),
        }


def _token(value, what: str) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value < 0:
        raise ValueError(f"{what} must hold non-negative integers")
    return value


class Request:
    """`consumed` counts the prompt tokens that are in the cache; a request decodes once its
    whole prompt is consumed.  The last generated token is never fed back, so at most
    prompt + max_new_tokens - 1 tokens are ever cached (scheduler.py:52-55 of the reference)."""

    def __init__(
        self,
        request_id: str,
        prompt: Sequence[int],
        *,
        max_new_tokens: int,
        stop_tokens=None,
        sampling: SamplingParams = GREEDY,
        order: int = 0,
    ) -> None:
        if not request_id:
            raise ValueError("request_id must not be empty")
        tokens = tuple(prompt)
        if not tokens:
            raise ValueError("the prompt must not be empty")
        if isinstance(max_new_tokens, bool) or not isinstance(max_new_tokens, int) or max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be a positive integer")
        if not isinstance(sampling, SamplingParams):
            raise ValueError("sampling must be a SamplingParams")
        if stop_tokens is None:
            stop_tokens = ()
        elif isinstance(stop_tokens, int):
            stop_tokens = (stop_tokens,)
        self.id = request_id
        self.prompt = tuple(_token(t, "the prompt") for t in tokens)
        self.max_new_tokens = max_new_tokens
        self.stop_tokens = frozenset(_token(t, "eos_token_ids") for t in stop_tokens)
        self.sampling = sampling
        self.order = order
        self.phase = Phase.QUEUED
        self.consumed = 0
        self.output: list[int] = []
        self.end_reason: Optional[EndReason] = None
        self.timeline = Timeline()

    def __repr__(self) -> str:
        return f"Request({self.id!r}, {self.phase.value}, consumed {self.consumed}/{len(self.prompt)}, {len(self.output)} out)"

    @property
    def generated(self) -> tuple[int, ...]:
        return tuple(self.output)

    @property
    def prompt_left(self) -> int:
        return len(self.prompt) - self.consumed

    @property
    def decoding(self) -> bool:
        return self.consumed == len(self.prompt)

    @property
    def cache_tokens(self) -> int:
        """Most tokens this request ever holds in the cache."""
        return len(self.prompt) + self.max_new_tokens - 1

    @property
    def untouched(self) -> bool:
        return self.consumed == 0 and not self.output

    def accept(self, token: int) -> Optional[EndReason]:
        """Take a generated token; says whether (and why) the request ends with it.  A stop
        token ends it even when the length would too."""
        self.output.append(token)
        if token in self.stop_tokens:
            self.end_reason = EndReason.STOP_TOKEN
        elif len(self.output) >= self.max_new_tokens:
            self.end_reason = EndReason.LENGTH
        return self.end_reason
