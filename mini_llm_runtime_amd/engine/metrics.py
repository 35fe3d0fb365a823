"""Figures of finished and running requests, read from their timelines."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Iterable, Optional

from .request import Request


@dataclass(frozen=True)
class RequestTimes:
    """queue wait, time to first token, median time between tokens, end to end (from the
    arrival to the last token) and the clean-up after it, in milliseconds; None where the
    request has not got that far (definitions: `engine.request.Timeline`)."""

    request_id: str
    tokens: int
    queue_wait_ms: Optional[float]
    ttft_ms: Optional[float]
    median_tpot_ms: Optional[float]
    e2e_ms: Optional[float]
    cleanup_ms: Optional[float]

    @staticmethod
    def of(request: Request) -> "RequestTimes":
        return RequestTimes(request.id, len(request.output), **request.timeline.figures_ms())


def summarize(requests: Iterable[Request]) -> dict[str, Optional[float]]:
    """Medians over requests of time to first token and of their median time between tokens."""
    times = [RequestTimes.of(r) for r in requests]

    def median(values):
        values = sorted(v for v in values if v is not None)
        return values[len(values) // 2] if values else None

    return {
        "requests": len(times),
        "median_ttft_ms": median(t.ttft_ms for t in times),
        "median_tpot_ms": median(t.median_tpot_ms for t in times),
        "median_e2e_ms": median(t.e2e_ms for t in times),
    }
