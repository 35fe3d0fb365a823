"""The continuous-batching loop: plan a step, run it, choose tokens, apply them, give pages back.

What one step does follows the reference's engine (src/mini_llm_runtime/engine.py:150-281): the
scheduler decides; the model runs; tokens are chosen on the GPU and come to the host in ONE
copy (engine.py:257-261); the results are applied and finished requests' pages are released in
the same step (engine.py:268-269).  When anything fails, the requests the plan admitted are
released and the plan is cancelled, so that the same step can be tried again
(engine.py:249-254).  Unlike the reference, which runs prompts and decodes as two forwards
(engine.py:186-248), a step here is one forward over the whole batch, and the plan's entries
go to the step function as they are.

Decoding one step ahead.  The host's share of a decode step (planning, block tables, the
launch itself, waiting for the chosen tokens) is a good part of the step's time for a small
model, and the GPU would idle through it.  So, before it waits for the tokens of step k, the
engine launches step k+1 for the same requests with the token ids taken on the device from
the sampler's output; nothing about that step counts yet.  When the scheduler, now knowing
step k's tokens, plans exactly that step, it is committed and only its tokens are waited for;
when it plans anything else (a request finished, another was admitted) the launch is
abandoned: its pages go back, and what it wrote is overwritten by the steps that follow it on
the stream.  Results, their order and the scheduler's decisions are those of the plain loop.
"""

from __future__ import annotations

import time
import warnings
from contextlib import contextmanager
from dataclasses import dataclass
from pathlib import Path
from typing import Callable, Collection, Iterator, Optional, Sequence, Union

import torch

from ..sampling.sampler import GREEDY, Sampler, SamplingParams
from .admission import PageAdmission
from .config import EngineConfig
from .metrics import RequestTimes
from .request import Request
from .runner import ModelRunner, StepOutput
from .scheduler import Scheduler, StepPlan, StepReport


@contextmanager
def _traced(enabled: bool, label: str) -> Iterator[None]:
    """A named range for rocprofv3's marker trace; closed on errors too.  The names are the
    reference's (engine.py:24-33, 170-281), so that traces of both read alike."""
    if enabled:
        torch.cuda.nvtx.range_push(label)
    try:
        yield
    finally:
        if enabled:
            torch.cuda.nvtx.range_pop()


class _ChosenTokens:
    """The tokens chosen in one step, on their way to the host.  The copy is put on the stream
    right behind the sampling, BEFORE any later step is launched, and has an event of its own:
    waiting for it does not wait for what was launched after it."""

    def __init__(self, on_device: torch.Tensor, spare: list) -> None:
        """spare: the engine's pinned landing buffers that are not in use (making one costs a
        system call); this object takes one and puts it back in `wait`."""
        self.on_device = on_device
        self._event = self._buffer = None
        self._spare = spare
        if on_device.device.type != "cuda":
            self._host = on_device
            return
        count = on_device.numel()
        self._buffer = spare.pop() if spare and spare[-1].numel() >= count else torch.empty(
            max(256, count), dtype=on_device.dtype, pin_memory=True
        )
        self._host = self._buffer[:count]
        self._host.copy_(on_device, non_blocking=True)
        self._event = torch.cuda.Event()
        self._event.record(torch.cuda.current_stream(on_device.device))

    def wait(self) -> list[int]:
        if self._event is not None:
            self._event.synchronize()
        tokens = self._host.tolist()
        if self._buffer is not None and len(self._spare) < 8:
            self._spare.append(self._buffer)
        self._buffer = None
        return tokens


class EngineBrokenError(RuntimeError):
    """A step failed after the cache had counted its tokens (while tokens were chosen or copied):
    scheduler and cache no longer agree, and no further step may run."""


@dataclass
class _Flight:
    """A step that has been launched: what the step function returned and the chosen tokens."""

    request_ids: tuple[str, ...]
    output: StepOutput
    chosen: Optional[_ChosenTokens]


@dataclass(frozen=True)
class EngineStepResult:
    plan: StepPlan
    report: StepReport
    released_blocks: tuple[tuple[str, dict], ...]  # (request, pages it held per pool) of the requests that ended
    started_ns: int
    tokens_ready_ns: int
    completed_ns: int


class ContinuousBatchEngine:
    def __init__(
        self,
        *,
        scheduler: Scheduler,
        runner: ModelRunner,
        admission: PageAdmission,
        sampler: Optional[Sampler] = None,
        clock_ns: Callable[[], int] = time.perf_counter_ns,
        enable_tracing: bool = False,
        lookahead: bool = True,
    ) -> None:
        if admission.manager is not runner.cache:
            raise ValueError("the admission and the runner must share one cache manager")
        if scheduler.max_running_requests > runner.cache.max_requests:
            raise ValueError("the scheduler may run more requests than the cache manager has slots")
        if scheduler.cut_prompts and not runner.model.splittable:
            raise ValueError("a part of this model needs whole prompts: the scheduler must not cut them (cut_prompts=False)")
        if enable_tracing and runner.device.type != "cuda":
            raise ValueError("tracing ranges need a GPU engine")
        self.scheduler = scheduler
        self.runner = runner
        self.admission = admission
        self.sampler = sampler or Sampler(runner.ops, runner.device)
        self._clock_ns = clock_ns
        self.enable_tracing = enable_tracing
        self.lookahead = bool(lookahead)
        self._ahead: Optional[_Flight] = None
        self.lookahead_hits = 0
        self.lookahead_misses = 0
        self.lookahead_error: Optional[Exception] = None  # what switched the lookahead off, if anything did
        self.broken: Optional[BaseException] = None  # what failed after a step's tokens had been counted
        self._landing: list = []  # pinned buffers for chosen tokens that are not in use
        self.config: Optional[EngineConfig] = None  # set by from_model_dir

    @property
    def manager(self):
        return self.admission.manager

    # ---- from a model folder --------------------------------------------------------------------
    @classmethod
    def from_model_dir(
        cls,
        model_dir: Union[str, Path],
        config: Optional[EngineConfig] = None,
        *,
        ops=None,
        **overrides,
    ) -> "ContinuousBatchEngine":
        """Model folder -> engine, set up by an `EngineConfig` (keyword arguments replace
        single fields of it).  `ops` replaces the HIP kernel library (tests on the CPU)."""
        from ..config.model_config import read_config_json
        from ..models.registry import load_config
        from .factory import blocks_from_free_memory, default_ops, load_model, make_cache, recording_reserve_bytes

        config = (config or EngineConfig()).with_overrides(**overrides)
        dtype = ops.dtype if ops is not None and config.dtype is None else config.resolved_dtype(read_config_json(model_dir))
        ops = ops or default_ops(dtype, config.device, config.tuning)
        load_config(model_dir)  # an unknown architecture fails before any weight is read
        _, model = load_model(model_dir, dtype=dtype, device=ops.device)
        num_blocks = config.num_blocks
        if num_blocks is None:
            reserve = recording_reserve_bytes(
                model, config.graphs, dtype, config.max_running_requests, config.max_batch_tokens
            )
            num_blocks = blocks_from_free_memory(
                model, config.block_size, dtype, torch.device(ops.device), config.kv_memory_fraction, reserve
            )
        cache = make_cache(
            model,
            block_size=config.block_size,
            num_blocks=num_blocks,
            max_requests=config.max_running_requests,
            check_visibility=config.check_cache_visibility,
        )
        limits = config.graphs
        runner = ModelRunner(
            model,
            cache,
            ops,
            use_graphs=limits.enabled,
            max_graph_batch=limits.max_decode_batch,
            max_decode_graphs=limits.max_decode_graphs,
            max_step_graphs=limits.max_step_graphs,
            max_graph_tokens=limits.max_step_tokens,
        )
        admission = PageAdmission(cache, max_step_tokens=config.max_batch_tokens)
        scheduler = Scheduler(
            max_running_requests=config.max_running_requests,
            max_batch_tokens=config.max_batch_tokens,
            max_mixed_prefill_tokens=config.max_mixed_prefill_tokens,
            admit=admission.admit,
            batching_policy=config.batching_policy,
            cut_prompts=model.splittable,  # a capability of the model's parts, not a choice of the caller
        )
        engine = cls(
            scheduler=scheduler,
            runner=runner,
            admission=admission,
            enable_tracing=config.enable_tracing,
            lookahead=config.lookahead,
        )
        engine.config = config
        return engine

    # ---- requests -------------------------------------------------------------------------------
    def submit(
        self,
        request_id: str,
        prompt_token_ids: Sequence[int],
        *,
        max_new_tokens: int,
        eos_token_ids: Union[int, Collection[int], None] = None,
        temperature: float = 0.0,
        seed: int = 0,
    ) -> Request:
        """Queue a request (names of the reference's entry point, engine.py:120-148).  Refused
        here, before it is queued: tokens outside the vocabulary, more positions than the model
        has, and a request that no empty page pool could hold (it would sit at the head of the
        queue for good, and everything behind it with it)."""
        arrived = self._clock_ns()
        vocab = self.runner.vocab_size
        outside = [t for t in prompt_token_ids if isinstance(t, int) and t >= vocab]
        if outside:
            raise ValueError(f"prompt tokens outside the vocabulary of {vocab}: {outside[:5]}")
        lifetime = len(prompt_token_ids) + max_new_tokens - 1
        if lifetime > self.runner.max_positions:
            raise ValueError("prompt length + max_new_tokens - 1 exceeds max_position_embeddings")
        if not self.admission.can_ever_admit(lifetime):
            have = [g.num_blocks for g in self.manager.groups]
            raise ValueError(
                f"request {request_id!r} can never be admitted: it needs {list(self.admission.pages_for(lifetime))} "
                f"pages per pool, the pools have {have}"
            )
        sampling = GREEDY if temperature == 0.0 else SamplingParams(float(temperature), int(seed))
        request = self.scheduler.add(
            request_id, prompt_token_ids, max_new_tokens=max_new_tokens, stop_tokens=eos_token_ids, sampling=sampling
        )
        request.timeline.stamp("arrived", arrived)
        return request

    def request(self, request_id: str) -> Request:
        return self.scheduler.request(request_id)

    def times(self, request_id: str) -> RequestTimes:
        return RequestTimes.of(self.scheduler.request(request_id))

    def all_times(self) -> tuple[RequestTimes, ...]:
        return tuple(RequestTimes.of(r) for r in self.scheduler.requests)

    # ---- one step -------------------------------------------------------------------------------
    @torch.inference_mode()
    def step(self) -> Optional[EngineStepResult]:
        """Plan and run one step; None when nothing can run."""
        if self.broken is not None:
            raise EngineBrokenError(
                f"an earlier step failed after the cache had counted its tokens ({type(self.broken).__name__}: "
                f"{self.broken}); the engine cannot go on"
            )
        started = self._clock_ns()
        try:
            with _traced(self.enable_tracing, "scheduler.schedule_step"):
                plan = self.scheduler.plan()
        except BaseException:
            self._abandon_ahead()  # whatever the scheduler refused, no launched step stays open
            raise
        if plan is None:
            self._abandon_ahead()
            return None
        label = f"engine.step:{plan.index}:prefill={len(plan.prompt_ids)}:decode={len(plan.decode_ids)}"
        with _traced(self.enable_tracing, label):
            try:
                flight = self._fly(plan)
            except EngineBrokenError:
                raise
            except BaseException:  # an interrupt, too, must not leave admitted requests and a plan behind
                self._abandon_ahead()
                with _traced(self.enable_tracing, "engine.rollback"):
                    self.admission.release(plan.admitted)
                    self.scheduler.cancel()
                raise
            if self.lookahead and flight.chosen is not None:
                self._look_ahead(plan, flight)
            with _traced(self.enable_tracing, "token.d2h_sync"):
                tokens = flight.chosen.wait() if flight.chosen is not None else []
            ready = self._clock_ns()
            with _traced(self.enable_tracing, "scheduler.apply_and_release"):
                report = self.scheduler.complete({rid: int(t) for (rid, _), t in zip(flight.output.rows, tokens)})
                if self._ahead is not None and set(report.finished) & set(self._ahead.request_ids):
                    self._abandon_ahead()  # it holds pages of a request that is about to be released
                released = self.admission.release(report.finished)
            completed = self._clock_ns()
        for rid, _ in report.emitted:
            self.scheduler.request(rid).timeline.stamp("token", ready)
        for rid in report.finished:
            self.scheduler.request(rid).timeline.stamp("done", completed)
        return EngineStepResult(plan, report, tuple(released.items()), started, ready, completed)

    def _sampling_of(self, plan: StepPlan) -> tuple[list[SamplingParams], list[int]]:
        """Sampling parameters and index of the token to come, for every slice that emits one."""
        emitting = [s.request for s in plan.slices if s.emits]
        return [r.sampling for r in emitting], [len(r.output) for r in emitting]

    def _fly(self, plan: StepPlan) -> _Flight:
        """Launch the plan's step: the one launched ahead if it is that step, else a new one."""
        for part in plan.slices:
            if part.from_prompt and part.offset == 0:
                part.request.timeline.stamp("scheduled", self._clock_ns())
        ahead = self._ahead
        if ahead is not None:
            same = not plan.admitted and not plan.prompt_ids and plan.decode_ids == ahead.request_ids
            if same:
                self._ahead = None
                self.lookahead_hits += 1
                ahead.output = self.runner.commit(ahead.output)
                return ahead
            self._abandon_ahead()
        self._check_offsets(plan)
        with _traced(self.enable_tracing, f"model.step:tokens={plan.token_count}"):
            output = self.runner.step(plan.entries, borrow_logits=True)  # sampled from right below
        # From here on the cache counts the step's tokens: a failure can no longer be undone by
        # cancelling the plan (the same tokens would be fed again behind themselves).
        try:
            chosen = None
            if output.logits is not None:
                chosen = _ChosenTokens(self.sampler.sample(output.logits, *self._sampling_of(plan)), self._landing)
        except BaseException as error:
            self.broken = error
            self._abandon_ahead()
            raise EngineBrokenError(
                f"choosing the tokens of step {plan.index} failed after the cache had counted them: "
                f"{type(error).__name__}: {error}"
            ) from error
        return _Flight(tuple(rid for rid, _ in output.rows), output, chosen)

    def _check_offsets(self, plan: StepPlan) -> None:
        """Every slice goes on exactly where its request's cache ends: the scheduler's count of
        consumed tokens and the cache manager's count of cached ones must agree."""
        for part in plan.slices:
            cached = self.manager.get_request(part.request_id).num_tokens
            if cached != part.offset:
                raise RuntimeError(
                    f"request {part.request_id!r}: the plan feeds tokens behind {part.offset} cached ones, "
                    f"the cache holds {cached}"
                )

    # ---- the step launched ahead ------------------------------------------------------------------
    def _look_ahead(self, plan: StepPlan, flight: _Flight) -> None:
        """Launch the next step now if it is bound to be one token for each request of this step
        that goes on: every active request emits a token here, nobody waits who could be let in,
        and those that end by length with this token are left out.  (A request may still end on a
        stop token; then the launch is abandoned.)  A failure here must not undo the step that is
        already launched and counted: decoding goes on without looking ahead."""
        try:
            with _traced(self.enable_tracing, "model.step:ahead"):
                self._ahead = self._launch_ahead(plan, flight)
        except Exception as error:  # noqa: BLE001
            self._ahead = None
            self.lookahead = False
            self.lookahead_error = error
            warnings.warn(
                f"decoding one step ahead was switched off after {type(error).__name__}: {error}; "
                "steps go on one by one, which is slower",
                RuntimeWarning,
                stacklevel=2,
            )

    def _launch_ahead(self, plan: StepPlan, flight: _Flight) -> Optional[_Flight]:
        scheduler = self.scheduler
        active = scheduler.active_ids
        emitting = plan.emitting_ids
        if not active or sorted(active) != sorted(emitting):
            return None
        if scheduler.queued_ids and len(active) < scheduler.max_running_requests:
            return None
        place = {rid: i for i, rid in enumerate(emitting)}
        going_on = [rid for rid in active if len(scheduler.request(rid).output) + 1 < scheduler.request(rid).max_new_tokens]
        if not going_on:
            return None
        picks = [place[rid] for rid in going_on]
        tokens = flight.chosen.on_device
        if picks != list(range(len(emitting))):
            tokens = tokens[torch.tensor(picks, dtype=torch.int64, device=tokens.device)]
        launched = self.runner.launch_decode(going_on, tokens)
        if launched is None:
            return None
        try:
            requests = [scheduler.request(rid) for rid in going_on]
            chosen = _ChosenTokens(
                self.sampler.sample(launched.logits, [r.sampling for r in requests], [len(r.output) + 1 for r in requests]),
                self._landing,
            )
        except BaseException:
            self.runner.abort(launched)
            raise
        return _Flight(tuple(going_on), launched, chosen)

    def _abandon_ahead(self) -> None:
        if self._ahead is not None:
            ahead, self._ahead = self._ahead, None
            self.lookahead_misses += 1
            self.runner.abort(ahead.output)

    # ---- to the end -----------------------------------------------------------------------------------
    def run_until_done(self) -> list[EngineStepResult]:
        """Step until every submitted request has finished."""
        results = []
        while self.scheduler.busy:
            result = self.step()
            if result is None:
                raise RuntimeError("requests are unfinished but nothing can run: the page budget admits no progress")
            results.append(result)
        return results

    def generate(
        self,
        prompts: Sequence[Sequence[int]],
        *,
        max_new_tokens: int,
        eos_token_ids: Union[int, Collection[int], None] = None,
        temperature: float = 0.0,
        seed: int = 0,
    ) -> list[list[int]]:
        """Submit all prompts, run to completion, return each prompt's generated tokens."""
        base = len(self.scheduler.requests)
        ids = [f"generate-{base + i}" for i in range(len(prompts))]
        for i, (rid, prompt) in enumerate(zip(ids, prompts)):
            self.submit(
                rid, list(prompt), max_new_tokens=max_new_tokens, eos_token_ids=eos_token_ids,
                temperature=temperature, seed=seed + i,
            )
        self.run_until_done()
        return [list(self.scheduler.request(rid).output) for rid in ids]
