"""The request state machine above the step function: waiting -> running -> finished.

Policy, as the reference's `RequestScheduler`
(src/mini_llm_runtime/scheduler.py:96-397): running requests decode first, one
token each; what is left of the token budget goes to prompts, strictly first come
first served; one batch is outstanding at a time; `schedule_step` and
`apply_step_results` alternate; an aborted step puts newly admitted requests back
at the front of the queue and keeps its step index.  STATIC batching admits only
when nothing is running, CONTINUOUS whenever there is room.

Beyond the reference: prompts are cut into portions under the token budget (the
reference refuses a prompt longer than the budget, scheduler.py:181-185).  A
request keeps `num_computed_tokens`; it takes min(rest of its prompt, rest of the
budget) tokens per step, a portion may be a single token, and it produces a
token only in the step that consumes the end of its prompt.

When pages run out: a request is admitted only if the pages of its whole life
(prompt + max_new_tokens - 1 tokens) can be promised to it, so a running request
never fails to grow; a request that does not fit waits at the head of the queue
and everything behind it waits too (scheduler.py:258-262, block_admission.py:35-67).
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from enum import Enum
from typing import Callable, Collection, Mapping, Optional, Sequence, Union

from ..sampling.sampler import GREEDY, SamplingParams


class RequestStatus(str, Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


class FinishReason(str, Enum):
    EOS = "eos"
    MAX_TOKENS = "max_tokens"


class WorkKind(str, Enum):
    PREFILL = "prefill"
    DECODE = "decode"


class BatchingPolicy(str, Enum):
    CONTINUOUS = "continuous"
    STATIC = "static"


@dataclass
class RequestState:
    request_id: str
    prompt_token_ids: tuple[int, ...]
    max_new_tokens: int
    eos_token_ids: frozenset[int]
    arrival_index: int
    sampling: SamplingParams = GREEDY
    status: RequestStatus = RequestStatus.WAITING
    num_computed_tokens: int = 0
    finish_reason: Optional[FinishReason] = None
    _generated_token_ids: list[int] = field(default_factory=list, repr=False)

    @property
    def generated_token_ids(self) -> tuple[int, ...]:
        return tuple(self._generated_token_ids)

    @property
    def prefilled(self) -> bool:
        return self.num_computed_tokens >= len(self.prompt_token_ids)

    @property
    def max_cache_tokens(self) -> int:
        # the last generated token is never fed back, so it is never cached
        # (scheduler.py:52-55 of the reference)
        return len(self.prompt_token_ids) + self.max_new_tokens - 1


@dataclass(frozen=True)
class ScheduledRequest:
    request_id: str
    kind: WorkKind
    input_token_ids: tuple[int, ...]
    start: int  # tokens of this request that are cached before the step
    produces_token: bool

    @property
    def token_cost(self) -> int:
        return len(self.input_token_ids)


@dataclass(frozen=True)
class SchedulerBatch:
    step_index: int
    items: tuple[ScheduledRequest, ...]
    token_count: int
    admitted_request_ids: tuple[str, ...] = ()

    @property
    def prefill_request_ids(self) -> tuple[str, ...]:
        return tuple(i.request_id for i in self.items if i.kind is WorkKind.PREFILL)

    @property
    def decode_request_ids(self) -> tuple[str, ...]:
        return tuple(i.request_id for i in self.items if i.kind is WorkKind.DECODE)

    @property
    def producing_request_ids(self) -> tuple[str, ...]:
        return tuple(i.request_id for i in self.items if i.produces_token)


@dataclass(frozen=True)
class SchedulerStepUpdate:
    step_index: int
    emitted_tokens: tuple[tuple[str, int], ...]
    finished_request_ids: tuple[str, ...]


class RequestScheduler:
    def __init__(
        self,
        *,
        max_running_requests: int,
        max_batch_tokens: int,
        max_mixed_prefill_tokens: Optional[int] = None,
        admission_callback: Optional[Callable[[RequestState], bool]] = None,
        batching_policy: BatchingPolicy = BatchingPolicy.CONTINUOUS,
        chunked_prefill: bool = True,
    ) -> None:
        if max_running_requests <= 0 or max_batch_tokens <= 0:
            raise ValueError("max_running_requests and max_batch_tokens must be > 0")
        if max_running_requests > max_batch_tokens:
            raise ValueError(
                "max_running_requests must not exceed max_batch_tokens, "
                "or running requests could not all decode in one step"
            )
        if not isinstance(batching_policy, BatchingPolicy):
            raise ValueError("batching_policy must be a BatchingPolicy")
        if max_mixed_prefill_tokens is not None and (
            isinstance(max_mixed_prefill_tokens, bool)
            or not isinstance(max_mixed_prefill_tokens, int)
            or max_mixed_prefill_tokens <= 0
        ):
            raise ValueError("max_mixed_prefill_tokens must be a positive integer or None")
        self.max_running_requests = max_running_requests
        self.max_batch_tokens = max_batch_tokens
        self.max_mixed_prefill_tokens = max_mixed_prefill_tokens
        self.batching_policy = batching_policy
        self.chunked_prefill = bool(chunked_prefill)
        self._admission_callback = admission_callback
        self._requests: dict[str, RequestState] = {}
        self._waiting: deque[str] = deque()
        self._running: list[str] = []
        self._finished: list[str] = []
        self._next_arrival_index = 0
        self._next_step_index = 0
        self._outstanding: Optional[SchedulerBatch] = None

    # ---- views ------------------------------------------------------------------------
    @property
    def waiting_request_ids(self) -> tuple[str, ...]:
        return tuple(self._waiting)

    @property
    def running_request_ids(self) -> tuple[str, ...]:
        return tuple(self._running)

    @property
    def finished_request_ids(self) -> tuple[str, ...]:
        return tuple(self._finished)

    @property
    def outstanding_batch(self) -> Optional[SchedulerBatch]:
        return self._outstanding

    @property
    def has_unfinished_requests(self) -> bool:
        return bool(self._waiting or self._running or self._outstanding)

    def get_request(self, request_id: str) -> RequestState:
        try:
            return self._requests[request_id]
        except KeyError:
            raise KeyError(f"unknown request_id={request_id!r}") from None

    # ---- arrivals ------------------------------------------------------------------------
    def submit(
        self,
        request_id: str,
        prompt_token_ids: Sequence[int],
        *,
        max_new_tokens: int,
        eos_token_ids: Union[int, Collection[int], None] = None,
        sampling: SamplingParams = GREEDY,
    ) -> RequestState:
        """Append a request to the end of the waiting queue."""
        if not request_id:
            raise ValueError("request_id must not be empty")
        if request_id in self._requests:
            raise ValueError(f"request_id={request_id!r} already exists")
        prompt = self._validate_token_sequence(prompt_token_ids, "prompt_token_ids")
        if not self.chunked_prefill and len(prompt) > self.max_batch_tokens:
            raise ValueError(
                f"prompt length={len(prompt)} exceeds max_batch_tokens={self.max_batch_tokens} "
                "and prompts are not cut into portions (chunked_prefill=False)"
            )
        if isinstance(max_new_tokens, bool) or not isinstance(max_new_tokens, int) or max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be a positive integer")
        if not isinstance(sampling, SamplingParams):
            raise ValueError("sampling must be a SamplingParams")
        request = RequestState(
            request_id=request_id,
            prompt_token_ids=prompt,
            max_new_tokens=int(max_new_tokens),
            eos_token_ids=self._normalize_eos(eos_token_ids),
            arrival_index=self._next_arrival_index,
            sampling=sampling,
        )
        self._next_arrival_index += 1
        self._requests[request_id] = request
        self._waiting.append(request_id)
        return request

    # ---- one step ---------------------------------------------------------------------------
    def schedule_step(self) -> Optional[SchedulerBatch]:
        """Decodes of all running requests first, then prompt portions, first come first served."""
        if self._outstanding is not None:
            raise RuntimeError("the previous batch's results were not applied yet")
        if not self._running and not self._waiting:
            return None

        items: list[ScheduledRequest] = []
        running_at_step_start = bool(self._running)
        for request_id in self._running:
            request = self._requests[request_id]
            if not request.prefilled:
                continue
            if not request._generated_token_ids:
                raise RuntimeError(f"running request {request_id!r} has consumed its prompt but produced no token")
            items.append(
                ScheduledRequest(
                    request_id=request_id,
                    kind=WorkKind.DECODE,
                    input_token_ids=(request._generated_token_ids[-1],),
                    start=len(request.prompt_token_ids) + len(request._generated_token_ids) - 1,
                    produces_token=True,
                )
            )
        token_count = len(items)
        mixed = bool(items)
        prompt_tokens = 0

        def room() -> int:
            left = self.max_batch_tokens - token_count
            if mixed and self.max_mixed_prefill_tokens is not None:
                left = min(left, self.max_mixed_prefill_tokens - prompt_tokens)
            return left

        def portion(request: RequestState) -> Optional[ScheduledRequest]:
            rest = len(request.prompt_token_ids) - request.num_computed_tokens
            take = min(rest, room())
            if take <= 0 or (not self.chunked_prefill and take < rest):
                return None
            begin = request.num_computed_tokens
            return ScheduledRequest(
                request_id=request.request_id,
                kind=WorkKind.PREFILL,
                input_token_ids=request.prompt_token_ids[begin : begin + take],
                start=begin,
                produces_token=begin + take == len(request.prompt_token_ids),
            )

        # running requests whose prompt is not consumed yet go on, oldest first
        blocked = False
        for request_id in self._running:
            request = self._requests[request_id]
            if request.prefilled:
                continue
            item = portion(request)
            if item is None:
                blocked = True
                break
            items.append(item)
            token_count += item.token_cost
            prompt_tokens += item.token_cost

        admitted: list[str] = []
        may_admit = self.batching_policy is BatchingPolicy.CONTINUOUS or not running_at_step_start
        while (
            may_admit
            and not blocked
            and self._waiting
            and len(self._running) < self.max_running_requests
        ):
            request = self._requests[self._waiting[0]]
            # strict FIFO: when the head does not fit, nobody behind it is looked at
            rest = len(request.prompt_token_ids)
            if room() <= 0 or (not self.chunked_prefill and rest > room()):
                break
            if self._admission_callback is not None and not self._admission_callback(request):
                break
            self._waiting.popleft()
            request.status = RequestStatus.RUNNING
            self._running.append(request.request_id)
            admitted.append(request.request_id)
            item = portion(request)
            assert item is not None
            items.append(item)
            token_count += item.token_cost
            prompt_tokens += item.token_cost

        if not items:
            return None
        batch = SchedulerBatch(
            step_index=self._next_step_index,
            items=tuple(items),
            token_count=token_count,
            admitted_request_ids=tuple(admitted),
        )
        self._next_step_index += 1
        self._outstanding = batch
        return batch

    def apply_step_results(self, generated_tokens: Mapping[str, int]) -> SchedulerStepUpdate:
        """Write back one token for every item that produced one; all or nothing."""
        batch = self._outstanding
        if batch is None:
            raise RuntimeError("no batch is waiting for results")
        expected = batch.producing_request_ids
        actual = tuple(generated_tokens)
        if set(actual) != set(expected) or len(actual) != len(expected):
            missing = sorted(set(expected) - set(actual))
            extra = sorted(set(actual) - set(expected))
            raise ValueError(f"step results do not match the batch: missing={missing}, extra={extra}")
        validated = {rid: self._validate_token(generated_tokens[rid], "generated token") for rid in expected}

        finished: list[str] = []
        emitted: list[tuple[str, int]] = []
        for item in batch.items:
            request = self._requests[item.request_id]
            if item.kind is WorkKind.PREFILL:
                request.num_computed_tokens += item.token_cost
            if not item.produces_token:
                continue
            token = validated[item.request_id]
            request._generated_token_ids.append(token)
            emitted.append((item.request_id, token))
            if token in request.eos_token_ids:
                request.finish_reason = FinishReason.EOS
            elif len(request._generated_token_ids) >= request.max_new_tokens:
                request.finish_reason = FinishReason.MAX_TOKENS
            if request.finish_reason is not None:
                request.status = RequestStatus.FINISHED
                finished.append(item.request_id)
        if finished:
            gone = set(finished)
            self._running = [rid for rid in self._running if rid not in gone]
            self._finished.extend(finished)
        self._outstanding = None
        return SchedulerStepUpdate(
            step_index=batch.step_index,
            emitted_tokens=tuple(emitted),
            finished_request_ids=tuple(finished),
        )

    def abort_step(self) -> SchedulerBatch:
        """Undo the outstanding batch so that the step can be tried again.

        Requests admitted by this batch return to the front of the queue in their
        order; requests that were already running changed nothing at scheduling
        time.  The cache is the engine's business (it releases the admitted
        requests before calling this).  The step index is used again.
        """
        batch = self._outstanding
        if batch is None:
            raise RuntimeError("no batch to abort")
        admitted = batch.admitted_request_ids
        for request_id in admitted:
            request = self._requests[request_id]
            if request.num_computed_tokens or request._generated_token_ids:
                raise RuntimeError(f"request {request_id!r} already has results and cannot be un-admitted")
            request.status = RequestStatus.WAITING
        gone = set(admitted)
        self._running = [rid for rid in self._running if rid not in gone]
        for request_id in reversed(admitted):
            self._waiting.appendleft(request_id)
        self._outstanding = None
        self._next_step_index = batch.step_index
        return batch

    # ---- validation ----------------------------------------------------------------------------
    @classmethod
    def _validate_token_sequence(cls, values: Sequence[int], name: str) -> tuple[int, ...]:
        tokens = tuple(values)
        if not tokens:
            raise ValueError(f"{name} must not be empty")
        return tuple(cls._validate_token(t, name) for t in tokens)

    @staticmethod
    def _validate_token(value: int, name: str) -> int:
        if isinstance(value, bool) or not isinstance(value, int) or value < 0:
            raise ValueError(f"{name} must hold non-negative integers")
        return value

    @classmethod
    def _normalize_eos(cls, values: Union[int, Collection[int], None]) -> frozenset[int]:
        if values is None:
            return frozenset()
        raw = (values,) if isinstance(values, int) else tuple(values)
        return frozenset(cls._validate_token(v, "eos_token_ids") for v in raw)
