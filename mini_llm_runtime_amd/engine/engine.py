"""The synchronous continuous-batching loop: scheduler -> step function -> sampler
-> scheduler, with pages given back as requests finish.

One engine step, as in the reference's `ContinuousBatchEngine.step`
(src/mini_llm_runtime/engine.py:150-281): schedule; run the model; choose tokens on
the GPU and bring them to the host in ONE copy (engine.py:257-261); apply the
results; release finished requests' pages in the same step (engine.py:268-269).
On any exception the step's newly admitted requests are released and the
scheduler's batch is undone, so the same step can be tried again
(engine.py:249-254).  Unlike the reference, which runs prompts and decodes as two
forwards (engine.py:186-248), a step here is one forward over the whole batch.

Decoding one step ahead.  The host's share of a decode step (scheduling, block
tables, the launch itself, waiting for the chosen tokens) is a good part of the
step's time for a small model, and the GPU would idle through it.  So, before it
waits for the tokens of step k, the engine launches step k+1 for the same requests
with the token ids taken on the device from the sampler's output; nothing about
that step counts yet.  When the scheduler, now knowing step k's tokens, asks for
exactly that step, it is committed and only its tokens are waited for; when it
asks for anything else (a request finished, another was admitted) the launch is
abandoned: its pages go back, and what it wrote is overwritten by the steps that
follow it on the stream.  Results, their order and the scheduler's decisions are
those of the plain loop.
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
from .admission import PagedBlockAdmissionController
from .config import EngineConfig
from .metrics import RequestMetricsCollector
from .runner import ModelRunner, StepEntry, StepOutput
from .scheduler import (
    BatchingPolicy,
    RequestScheduler,
    RequestState,
    SchedulerBatch,
    SchedulerStepUpdate,
    WorkKind,
)


@contextmanager
def _trace_range(enabled: bool, message: str) -> Iterator[None]:
    """Optional roctx range (visible to rocprofv3); always popped, also on errors."""
    if enabled:
        torch.cuda.nvtx.range_push(message)
    try:
        yield
    finally:
        if enabled:
            torch.cuda.nvtx.range_pop()


class _TokensOnTheWay:
    """The chosen tokens of one step, being copied to the host.  The copy is put on the
    stream right behind the sampling, BEFORE any later step is launched, and waited for by
    its own event: waiting for it then does not wait for what was launched after it."""

    _landing: list = []  # pinned host buffers that are not in use (allocating one costs a system call)

    def __init__(self, chosen: torch.Tensor) -> None:
        self.device_tokens = chosen
        self._event = None
        self._buffer = None
        if chosen.device.type == "cuda":
            count = chosen.numel()
            pool = _TokensOnTheWay._landing
            self._buffer = pool.pop() if pool and pool[-1].numel() >= count else torch.empty(
                max(256, count), dtype=chosen.dtype, pin_memory=True
            )
            self._host = self._buffer[:count]
            self._host.copy_(chosen, non_blocking=True)
            self._event = torch.cuda.Event()
            self._event.record(torch.cuda.current_stream(chosen.device))
        else:
            self._host = chosen

    def wait(self) -> list[int]:
        if self._event is not None:
            self._event.synchronize()
        tokens = self._host.tolist()
        if self._buffer is not None:
            if len(_TokensOnTheWay._landing) < 8:
                _TokensOnTheWay._landing.append(self._buffer)
            self._buffer = None
        return tokens


@dataclass
class _LaunchedAhead:
    request_ids: tuple[str, ...]
    output: "StepOutput"
    chosen: _TokensOnTheWay


@dataclass(frozen=True)
class EngineStepResult:
    batch: SchedulerBatch
    update: SchedulerStepUpdate
    released_blocks: tuple[tuple[str, dict], ...]
    started_ns: int
    tokens_ready_ns: int
    completed_ns: int


class ContinuousBatchEngine:
    def __init__(
        self,
        *,
        scheduler: RequestScheduler,
        runner: ModelRunner,
        admission: PagedBlockAdmissionController,
        sampler: Optional[Sampler] = None,
        clock_ns: Callable[[], int] = time.perf_counter_ns,
        metrics: Optional[RequestMetricsCollector] = None,
        enable_tracing: bool = False,
        lookahead: bool = True,
    ) -> None:
        if admission.manager is not runner.cache:
            raise ValueError("the admission controller and the runner must share one cache manager")
        if scheduler.max_running_requests > runner.cache.max_requests:
            raise ValueError("the scheduler may run more requests than the cache manager has slots")
        if enable_tracing and runner.device.type != "cuda":
            raise ValueError("tracing ranges need a GPU engine")
        self.scheduler = scheduler
        self.runner = runner
        self.admission = admission
        self.sampler = sampler or Sampler(runner.ops, runner.device)
        self._clock_ns = clock_ns
        self.metrics = metrics or RequestMetricsCollector()
        self.enable_tracing = enable_tracing
        self.lookahead = bool(lookahead)
        self._ahead: Optional[_LaunchedAhead] = None
        self.lookahead_hits = 0
        self.lookahead_misses = 0
        self.lookahead_error: Optional[Exception] = None  # what switched the lookahead off, if anything did
        self.config: Optional[EngineConfig] = None  # set by from_model_dir

    @property
    def manager(self):
        return self.admission.manager

    # ---- construction from a model folder ------------------------------------------------------
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
        from ..models.registry import load_config
        from ..config.model_config import read_config_json
        from .factory import blocks_from_free_memory, default_ops, load_model, make_cache

        config = (config or EngineConfig()).with_overrides(**overrides)
        dtype = ops.dtype if ops is not None and config.dtype is None else config.resolved_dtype(read_config_json(model_dir))
        ops = ops or default_ops(dtype, config.device, config.tuning)
        load_config(model_dir)  # an unknown architecture fails before any weight is read
        _, model = load_model(model_dir, dtype=dtype, device=ops.device)
        num_blocks = config.num_blocks
        if num_blocks is None:
            num_blocks = blocks_from_free_memory(
                model, config.block_size, dtype, torch.device(ops.device), config.kv_memory_fraction
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
        admission = PagedBlockAdmissionController(cache, max_step_tokens=config.max_batch_tokens)
        scheduler = RequestScheduler(
            max_running_requests=config.max_running_requests,
            max_batch_tokens=config.max_batch_tokens,
            max_mixed_prefill_tokens=config.max_mixed_prefill_tokens,
            admission_callback=admission.try_admit,
            batching_policy=config.batching_policy,
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

    # ---- requests ---------------------------------------------------------------------------------
    def submit(
        self,
        request_id: str,
        prompt_token_ids: Sequence[int],
        *,
        max_new_tokens: int,
        eos_token_ids: Union[int, Collection[int], None] = None,
        temperature: float = 0.0,
        seed: int = 0,
    ) -> RequestState:
        arrival_ns = self._clock_ns()
        vocab = self.runner.vocab_size
        bad = [t for t in prompt_token_ids if isinstance(t, int) and t >= vocab]
        if bad:
            raise ValueError(f"prompt tokens outside the vocabulary of {vocab}: {bad[:5]}")
        if len(prompt_token_ids) + max_new_tokens - 1 > self.runner.max_positions:
            raise ValueError("prompt length + max_new_tokens - 1 exceeds max_position_embeddings")
        # a request that no empty pool could hold would sit at the head of the queue for good,
        # and everything behind it with it: it is refused here, before it is queued
        lifetime = len(prompt_token_ids) + max_new_tokens - 1
        if not self.manager.can_ever_hold(lifetime, self.admission.max_step_tokens):
            need = self.manager.lifetime_blocks(lifetime, self.admission.max_step_tokens)
            have = [g.num_blocks for g in self.manager.groups]
            raise ValueError(
                f"request {request_id!r} can never be admitted: it needs {need} pages per pool, the pools have {have}"
            )
        sampling = GREEDY if temperature == 0.0 else SamplingParams(float(temperature), int(seed))
        request = self.scheduler.submit(
            request_id,
            prompt_token_ids,
            max_new_tokens=max_new_tokens,
            eos_token_ids=eos_token_ids,
            sampling=sampling,
        )
        self.metrics.register_request(request_id, arrival_ns)
        return request

    # ---- the loop -----------------------------------------------------------------------------------
    @torch.inference_mode()
    def step(self) -> Optional[EngineStepResult]:
        """Schedule and run one step; None when nothing can run."""
        started_ns = self._clock_ns()
        try:
            with _trace_range(self.enable_tracing, "scheduler.schedule_step"):
                batch = self.scheduler.schedule_step()
        except BaseException:
            self._drop_ahead()  # whatever the scheduler refused, no launched step stays open
            raise
        if batch is None:
            self._drop_ahead()
            return None
        label = (
            f"engine.step:{batch.step_index}:prefill={len(batch.prefill_request_ids)}:"
            f"decode={len(batch.decode_request_ids)}"
        )
        with _trace_range(self.enable_tracing, label):
            return self._execute(batch, started_ns)

    def _execute(self, batch: SchedulerBatch, started_ns: int) -> EngineStepResult:
        try:
            self.metrics.require_registered(tuple(i.request_id for i in batch.items))
            entries = []
            params: list[SamplingParams] = []
            indices: list[int] = []
            for item in batch.items:
                request = self.scheduler.get_request(item.request_id)
                if item.kind is WorkKind.PREFILL and item.start == 0:
                    self.metrics.record_prefill_started(item.request_id, self._clock_ns())
                want = (len(item.input_token_ids) - 1,) if item.produces_token else ()
                entries.append(StepEntry(item.request_id, item.input_token_ids, want))
                if item.produces_token:
                    params.append(request.sampling)
                    indices.append(len(request.generated_token_ids))
            ahead = self._take_ahead(batch)
            if ahead is not None:
                output = self.runner.commit(ahead.output)
                chosen = ahead.chosen
            else:
                with _trace_range(self.enable_tracing, f"model.step:tokens={batch.token_count}"):
                    output = self.runner.step(entries, borrow_logits=True)  # sampled from right below
                chosen = None
                if output.logits is not None:
                    chosen = _TokensOnTheWay(self.sampler.sample(output.logits, params, indices))
        except BaseException:  # also an interrupt must not leave admitted requests and a batch behind
            self._drop_ahead()
            with _trace_range(self.enable_tracing, "engine.rollback"):
                self.admission.release_admitted(batch.admitted_request_ids)
                self.scheduler.abort_step()
            raise

        if self.lookahead and chosen is not None:
            # step k is launched and counted; a failure to launch k+1 early must not undo it
            try:
                with _trace_range(self.enable_tracing, "model.step:ahead"):
                    self._ahead = self._launch_ahead(batch, output, chosen.device_tokens, params, indices)
            except Exception as error:  # noqa: BLE001 - decoding goes on without the lookahead
                self._ahead = None
                self.lookahead = False
                self.lookahead_error = error
                warnings.warn(
                    f"decoding one step ahead was switched off after {type(error).__name__}: {error}; "
                    "steps go on one by one, which is slower",
                    RuntimeWarning,
                    stacklevel=2,
                )
        with _trace_range(self.enable_tracing, "token.d2h_sync"):
            host_tokens = chosen.wait() if chosen is not None else []
        tokens_ready_ns = self._clock_ns()
        generated = {rid: int(tok) for (rid, _), tok in zip(output.rows, host_tokens)}
        with _trace_range(self.enable_tracing, "scheduler.apply_and_release"):
            update = self.scheduler.apply_step_results(generated)
            if self._ahead is not None and set(update.finished_request_ids) & set(self._ahead.request_ids):
                self._drop_ahead()  # it holds pages of a request that is about to be released
            released = self.admission.release_finished(update.finished_request_ids)
        completed_ns = self._clock_ns()
        self.metrics.record_tokens(update.emitted_tokens, tokens_ready_ns)
        self.metrics.record_completed(update.finished_request_ids, completed_ns)
        return EngineStepResult(
            batch=batch,
            update=update,
            released_blocks=tuple(released.items()),
            started_ns=started_ns,
            tokens_ready_ns=tokens_ready_ns,
            completed_ns=completed_ns,
        )

    # ---- the step launched ahead ----------------------------------------------------------------------
    def _launch_ahead(self, batch, output: StepOutput, chosen, params, indices) -> Optional[_LaunchedAhead]:
        """Launch the next step now if it is bound to be one token for each request of this
        batch that goes on: all running requests produced a token here, nobody waits who could
        be admitted, and those that end by length with this token are left out.  (A request may
        still end on an end-of-sequence token; then the launch is abandoned.)"""
        scheduler = self.scheduler
        running = scheduler.running_request_ids
        produced = [rid for rid, _ in output.rows]
        if not running or sorted(running) != sorted(produced):
            return None
        if scheduler.waiting_request_ids and len(running) < scheduler.max_running_requests:
            return None
        by_id = {rid: i for i, rid in enumerate(produced)}
        going_on = [rid for rid in running if indices[by_id[rid]] + 1 < scheduler.get_request(rid).max_new_tokens]
        if not going_on:
            return None
        order = [by_id[rid] for rid in going_on]
        tokens = chosen
        if order != list(range(len(produced))):
            tokens = chosen[torch.tensor(order, dtype=torch.int64, device=chosen.device)]
        launched = self.runner.launch_decode(going_on, tokens)
        if launched is None:
            return None
        try:
            ahead = _TokensOnTheWay(
                self.sampler.sample(launched.logits, [params[i] for i in order], [indices[i] + 1 for i in order])
            )
        except BaseException:
            self.runner.abort(launched)
            raise
        return _LaunchedAhead(tuple(going_on), launched, ahead)

    def _take_ahead(self, batch: SchedulerBatch) -> Optional[_LaunchedAhead]:
        """The step launched ahead if `batch` is that step; otherwise it is abandoned."""
        ahead = self._ahead
        if ahead is None:
            return None
        same = (
            not batch.admitted_request_ids
            and all(i.kind is WorkKind.DECODE for i in batch.items)
            and tuple(i.request_id for i in batch.items) == ahead.request_ids
        )
        if not same:
            self._drop_ahead()
            return None
        self._ahead = None
        self.lookahead_hits += 1
        return ahead

    def _drop_ahead(self) -> None:
        if self._ahead is not None:
            ahead, self._ahead = self._ahead, None
            self.lookahead_misses += 1
            self.runner.abort(ahead.output)

    def run_until_done(self) -> list[EngineStepResult]:
        """Step until every submitted request has finished."""
        results = []
        while self.scheduler.has_unfinished_requests:
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
        base = len(self.metrics.request_ids)
        ids = [f"generate-{base + i}" for i in range(len(prompts))]
        for i, (rid, prompt) in enumerate(zip(ids, prompts)):
            self.submit(
                rid,
                list(prompt),
                max_new_tokens=max_new_tokens,
                eos_token_ids=eos_token_ids,
                temperature=temperature,
                seed=seed + i,
            )
        self.run_until_done()
        return [list(self.scheduler.get_request(rid).generated_token_ids) for rid in ids]
