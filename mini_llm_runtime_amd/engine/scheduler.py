"""Which requests run in the next step, with which tokens.

The policy is the reference's (src/mini_llm_runtime/scheduler.py:96-397,
docs/scheduler_state_machine.md): requests that decode go first, one token each; what is
left of the token budget goes to prompts, strictly first come first served (when the head
of the queue does not fit, nobody behind it is looked at); one plan is outstanding at a
time; a cancelled plan puts the requests it admitted back at the front of the queue and
its index is used again.  STATIC batching admits only into an empty engine, CONTINUOUS
whenever there is room.

Beyond the reference: prompts are cut into portions under the token budget (the reference
refuses a prompt longer than the budget, scheduler.py:181-185).  A request takes
min(rest of its prompt, rest of the budget) tokens per step, a portion may be a single
token, and it produces a token only in the step that consumes the end of its prompt.
`cut_prompts=False` is for models whose parts cannot go on from a cached prefix.

When pages run out: `admit` (the page admission) lets a request in only if the pages of its
whole life can be promised to it, so an admitted request never fails to grow; one that does
not fit waits at the head of the queue and everything behind it waits too
(scheduler.py:258-262, block_admission.py:35-67).

A plan's `entries` are what the step function takes, as they are.
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass
from enum import Enum
from typing import Callable, Mapping, Optional, Sequence

from ..sampling.sampler import GREEDY, SamplingParams
from .request import Phase, Request
from .runner import StepEntry


class BatchingPolicy(str, Enum):
    CONTINUOUS = "continuous"
    STATIC = "static"


@dataclass(frozen=True)
class Slice:
    """One request's share of a step: `tokens` behind `offset` cached ones.  It emits a token
    when it holds the end of the prompt, or the token decoded last."""

    request: Request
    tokens: tuple[int, ...]
    offset: int
    emits: bool
    from_prompt: bool

    @property
    def request_id(self) -> str:
        return self.request.id

    @property
    def entry(self) -> StepEntry:
        return StepEntry(self.request.id, self.tokens, (len(self.tokens) - 1,) if self.emits else ())


@dataclass(frozen=True)
class StepPlan:
    index: int
    slices: tuple[Slice, ...]
    admitted: tuple[str, ...] = ()  # requests that entered with this plan

    @property
    def token_count(self) -> int:
        return sum(len(s.tokens) for s in self.slices)

    @property
    def entries(self) -> tuple[StepEntry, ...]:
        return tuple(s.entry for s in self.slices)

    @property
    def prompt_ids(self) -> tuple[str, ...]:
        return tuple(s.request.id for s in self.slices if s.from_prompt)

    @property
    def decode_ids(self) -> tuple[str, ...]:
        return tuple(s.request.id for s in self.slices if not s.from_prompt)

    @property
    def emitting_ids(self) -> tuple[str, ...]:
        return tuple(s.request.id for s in self.slices if s.emits)


@dataclass(frozen=True)
class StepReport:
    index: int
    emitted: tuple[tuple[str, int], ...]
    finished: tuple[str, ...]


class _Budget:
    """Tokens a step may still take; beside decoding requests prompts get at most `mixed_cap`."""

    def __init__(self, total: int, mixed_cap: Optional[int]) -> None:
        self.left = total
        self.mixed_cap = mixed_cap
        self.mixed = False
        self.prompt_tokens = 0

    def decode(self) -> None:
        self.left -= 1
        self.mixed = True

    def room_for_prompt(self) -> int:
        room = self.left
        if self.mixed and self.mixed_cap is not None:
            room = min(room, self.mixed_cap - self.prompt_tokens)
        return room

    def prompt(self, tokens: int) -> None:
        self.left -= tokens
        self.prompt_tokens += tokens


class Scheduler:
    def __init__(
        self,
        *,
        max_running_requests: int,
        max_batch_tokens: int,
        max_mixed_prefill_tokens: Optional[int] = None,
        admit: Optional[Callable[[Request], bool]] = None,
        batching_policy: BatchingPolicy = BatchingPolicy.CONTINUOUS,
        cut_prompts: bool = True,
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
        cap = max_mixed_prefill_tokens
        if cap is not None and (isinstance(cap, bool) or not isinstance(cap, int) or cap <= 0):
            raise ValueError("max_mixed_prefill_tokens must be a positive integer or None")
        self.max_running_requests = max_running_requests
        self.max_batch_tokens = max_batch_tokens
        self.max_mixed_prefill_tokens = cap
        self.batching_policy = batching_policy
        self.cut_prompts = bool(cut_prompts)
        self._admit = admit
        self._requests: dict[str, Request] = {}
        self._queue: deque[Request] = deque()
        self._active: list[Request] = []
        self._done: list[Request] = []
        self._next_index = 0
        self._pending: Optional[StepPlan] = None

    # ---- what is where ------------------------------------------------------------------------
    @property
    def queued_ids(self) -> tuple[str, ...]:
        return tuple(r.id for r in self._queue)

    @property
    def active_ids(self) -> tuple[str, ...]:
        return tuple(r.id for r in self._active)

    @property
    def done_ids(self) -> tuple[str, ...]:
        return tuple(r.id for r in self._done)

    @property
    def pending(self) -> Optional[StepPlan]:
        """The plan whose results have not come back yet."""
        return self._pending

    @property
    def busy(self) -> bool:
        return bool(self._queue or self._active or self._pending)

    @property
    def requests(self) -> tuple[Request, ...]:
        return tuple(self._requests.values())

    def request(self, request_id: str) -> Request:
        try:
            return self._requests[request_id]
        except KeyError:
            raise KeyError(f"unknown request {request_id!r}") from None

    # ---- arrivals -----------------------------------------------------------------------------
    def add(
        self,
        request_id: str,
        prompt: Sequence[int],
        *,
        max_new_tokens: int,
        stop_tokens=None,
        sampling: SamplingParams = GREEDY,
    ) -> Request:
        """Queue a new request behind the others."""
        if request_id in self._requests:
            raise ValueError(f"request {request_id!r} already exists")
        request = Request(
            request_id, prompt, max_new_tokens=max_new_tokens, stop_tokens=stop_tokens, sampling=sampling,
            order=len(self._requests),
        )
        if not self.cut_prompts and len(request.prompt) > self.max_batch_tokens:
            raise ValueError(
                f"a prompt of {len(request.prompt)} tokens exceeds max_batch_tokens={self.max_batch_tokens} "
                "and prompts are not cut into portions"
            )
        self._requests[request_id] = request
        self._queue.append(request)
        return request

    # ---- one step -----------------------------------------------------------------------------
    def _portion(self, request: Request, budget: _Budget) -> Optional[Slice]:
        """The next tokens of a request's prompt that fit, or None."""
        take = min(request.prompt_left, budget.room_for_prompt())
        if take <= 0 or (take < request.prompt_left and not self.cut_prompts):
            return None
        budget.prompt(take)
        first = request.consumed
        return Slice(request, request.prompt[first : first + take], first, take == request.prompt_left, True)

    def plan(self) -> Optional[StepPlan]:
        """The next step, or None when nothing can run."""
        if self._pending is not None:
            raise RuntimeError("the previous plan's results were not applied yet")
        if not self._active and not self._queue:
            return None
        budget = _Budget(self.max_batch_tokens, self.max_mixed_prefill_tokens)
        slices: list[Slice] = []
        was_empty = not self._active
        for request in self._active:  # decoding requests first
            if request.decoding:
                if not request.output:
                    raise RuntimeError(f"request {request.id!r} has consumed its prompt but produced no token")
                cached = len(request.prompt) + len(request.output) - 1
                slices.append(Slice(request, (request.output[-1],), cached, True, False))
                budget.decode()
        stuck = False
        for request in self._active:  # then prompts that are under way, oldest first
            if request.decoding:
                continue
            part = self._portion(request, budget)
            if part is None:
                stuck = True
                break
            slices.append(part)
        admitted: list[str] = []
        may_admit = not stuck and (self.batching_policy is BatchingPolicy.CONTINUOUS or was_empty)
        while may_admit and self._queue and len(self._active) < self.max_running_requests:
            head = self._queue[0]
            room = budget.room_for_prompt()
            if room <= 0 or (not self.cut_prompts and len(head.prompt) > room):
                break  # first come first served: nobody overtakes the head of the queue
            if self._admit is not None and not self._admit(head):
                break
            self._queue.popleft()
            head.phase = Phase.ACTIVE
            self._active.append(head)
            admitted.append(head.id)
            slices.append(self._portion(head, budget))
        if not slices:
            return None
        self._pending = StepPlan(self._next_index, tuple(slices), tuple(admitted))
        self._next_index += 1
        return self._pending

    def complete(self, tokens: Mapping[str, int]) -> StepReport:
        """The pending plan ran: one token for every slice that emits one; all or nothing."""
        plan = self._pending
        if plan is None:
            raise RuntimeError("no plan is waiting for results")
        expected = plan.emitting_ids
        if set(tokens) != set(expected) or len(tokens) != len(expected):
            missing = sorted(set(expected) - set(tokens))
            extra = sorted(set(tokens) - set(expected))
            raise ValueError(f"step results do not match the plan: missing={missing}, extra={extra}")
        for rid, token in tokens.items():
            if isinstance(token, bool) or not isinstance(token, int) or token < 0:
                raise ValueError(f"the token of {rid!r} must be a non-negative integer")
        emitted: list[tuple[str, int]] = []
        finished: list[Request] = []
        for part in plan.slices:
            request = part.request
            if part.from_prompt:
                request.consumed += len(part.tokens)
            if not part.emits:
                continue
            token = tokens[request.id]
            emitted.append((request.id, token))
            if request.accept(token) is not None:
                request.phase = Phase.DONE
                finished.append(request)
        if finished:
            self._active = [r for r in self._active if r.phase is not Phase.DONE]
            self._done.extend(finished)
        self._pending = None
        return StepReport(plan.index, tuple(emitted), tuple(r.id for r in finished))

    def cancel(self) -> StepPlan:
        """Undo the pending plan so that the step can be tried again: the requests it admitted
        return to the front of the queue in their order (the others changed nothing when the
        plan was made), and its index is used again.  The cache is the engine's business."""
        plan = self._pending
        if plan is None:
            raise RuntimeError("no plan to cancel")
        back = [self._requests[rid] for rid in plan.admitted]
        for request in back:
            if not request.untouched:
                raise RuntimeError(f"request {request.id!r} already has results and cannot be un-admitted")
            request.phase = Phase.QUEUED
        self._active = [r for r in self._active if r.phase is Phase.ACTIVE]
        self._queue.extendleft(reversed(back))
        self._pending = None
        self._next_index = plan.index
        return plan
