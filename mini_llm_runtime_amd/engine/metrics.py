"""Per-request timelines on one monotonic clock and the figures derived from them:
queue wait, time to first token, time between tokens, end-to-end time.

Definitions as in the reference (src/mini_llm_runtime/request_metrics.py:20-94): a
token's time is when the host can see it (after the device-to-host copy), TTFT and
E2E count from arrival, E2E ends at the last token, clean-up after it is reported
separately.
"""

from __future__ import annotations

import statistics
from dataclasses import dataclass, field
from typing import Optional

NS_PER_MS = 1_000_000


@dataclass(frozen=True)
class TokenEvent:
    token_id: int
    ready_ns: int


@dataclass(frozen=True)
class RequestMetrics:
    request_id: str
    arrival_ns: int
    prefill_attempt_started_ns: tuple[int, ...]
    token_events: tuple[TokenEvent, ...]
    completed_ns: Optional[int]

    @property
    def queue_wait_ns(self) -> Optional[int]:
        if not self.prefill_attempt_started_ns:
            return None
        return self.prefill_attempt_started_ns[0] - self.arrival_ns

    @property
    def ttft_ns(self) -> Optional[int]:
        return self.token_events[0].ready_ns - self.arrival_ns if self.token_events else None

    @property
    def inter_token_ns(self) -> tuple[int, ...]:
        ev = self.token_events
        return tuple(b.ready_ns - a.ready_ns for a, b in zip(ev, ev[1:]))

    @property
    def median_tpot_ns(self) -> Optional[float]:
        gaps = self.inter_token_ns
        return float(statistics.median(gaps)) if gaps else None

    @property
    def e2e_ns(self) -> Optional[int]:
        return self.token_events[-1].ready_ns - self.arrival_ns if self.token_events else None

    @property
    def post_token_completion_ns(self) -> Optional[int]:
        if self.completed_ns is None or not self.token_events:
            return None
        return self.completed_ns - self.token_events[-1].ready_ns

    @staticmethod
    def ns_to_ms(value) -> Optional[float]:
        return None if value is None else float(value) / NS_PER_MS

    @property
    def queue_wait_ms(self):
        return self.ns_to_ms(self.queue_wait_ns)

    @property
    def ttft_ms(self):
        return self.ns_to_ms(self.ttft_ns)

    @property
    def median_tpot_ms(self):
        return self.ns_to_ms(self.median_tpot_ns)

    @property
    def e2e_ms(self):
        return self.ns_to_ms(self.e2e_ns)


@dataclass
class _Timeline:
    arrival_ns: int
    prefill_attempt_started_ns: list[int] = field(default_factory=list)
    token_events: list[TokenEvent] = field(default_factory=list)
    completed_ns: Optional[int] = None

    def last_ns(self) -> int:
        times = [self.arrival_ns, *self.prefill_attempt_started_ns, *(e.ready_ns for e in self.token_events)]
        if self.completed_ns is not None:
            times.append(self.completed_ns)
        return max(times)


class RequestMetricsCollector:
    def __init__(self) -> None:
        self._timelines: dict[str, _Timeline] = {}

    @property
    def request_ids(self) -> tuple[str, ...]:
        return tuple(self._timelines)

    @staticmethod
    def _stamp(value: int) -> int:
        if isinstance(value, bool) or not isinstance(value, int) or value < 0:
            raise ValueError("a timestamp is a non-negative integer of nanoseconds")
        return value

    def _get(self, request_id: str) -> _Timeline:
        try:
            return self._timelines[request_id]
        except KeyError:
            raise KeyError(f"request {request_id!r} is not registered for metrics") from None

    def _forward(self, timeline: _Timeline, stamp: int) -> None:
        if self._stamp(stamp) < timeline.last_ns():
            raise ValueError("a request's events must not go back in time")

    def register_request(self, request_id: str, arrival_ns: int) -> None:
        if request_id in self._timelines:
            raise ValueError(f"request {request_id!r} is already registered")
        self._timelines[request_id] = _Timeline(self._stamp(arrival_ns))

    def require_registered(self, request_ids: tuple[str, ...]) -> None:
        missing = [rid for rid in request_ids if rid not in self._timelines]
        if missing:
            raise RuntimeError(f"requests must enter through engine.submit(): {missing}")

    def record_prefill_started(self, request_id: str, stamp: int) -> None:
        t = self._get(request_id)
        self._forward(t, stamp)
        if t.token_events or t.completed_ns is not None:
            raise RuntimeError("a request that produced tokens cannot start its prompt again")
        t.prefill_attempt_started_ns.append(stamp)

    def record_tokens(self, emitted: tuple[tuple[str, int], ...], stamp: int) -> None:
        if len({rid for rid, _ in emitted}) != len(emitted):
            raise ValueError("one token per request and step")
        timelines = [self._get(rid) for rid, _ in emitted]
        for t in timelines:
            self._forward(t, stamp)
            if t.completed_ns is not None:
                raise RuntimeError("a completed request cannot produce tokens")
        for (rid, token), t in zip(emitted, timelines):
            t.token_events.append(TokenEvent(int(token), stamp))

    def record_completed(self, request_ids: tuple[str, ...], stamp: int) -> None:
        timelines = [self._get(rid) for rid in request_ids]
        for t in timelines:
            self._forward(t, stamp)
            if t.completed_ns is not None:
                raise RuntimeError("the request is already completed")
            if not t.token_events:
                raise RuntimeError("a request without tokens cannot be completed")
        for t in timelines:
            t.completed_ns = stamp

    def snapshot(self, request_id: str) -> RequestMetrics:
        t = self._get(request_id)
        return RequestMetrics(
            request_id, t.arrival_ns, tuple(t.prefill_attempt_started_ns), tuple(t.token_events), t.completed_ns
        )

    def snapshots(self) -> tuple[RequestMetrics, ...]:
        return tuple(self.snapshot(rid) for rid in self._timelines)
