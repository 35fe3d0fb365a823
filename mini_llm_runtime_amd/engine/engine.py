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
"""

from __future__ import annotations

import time
from contextlib import contextmanager
from dataclasses import dataclass
from pathlib import Path
from typing import Callable, Collection, Iterator, Optional, Sequence, Union

import torch

from ..sampling.sampler import GREEDY, Sampler, SamplingParams
from .admission import PagedBlockAdmissionController
from .metrics import RequestMetricsCollector
from .runner import ModelRunner, StepEntry
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

    @property
    def manager(self):
        return self.admission.manager

    # ---- construction from a model folder ------------------------------------------------------
    @classmethod
    def from_model_dir(
        cls,
        model_dir: Union[str, Path],
        *,
        dtype: Union[str, torch.dtype] = "bfloat16",
        device: Union[str, torch.device] = "cuda",
        block_size: int = 16,
        num_blocks: int = 1024,
        max_running_requests: int = 8,
        max_batch_tokens: int = 2048,
        max_mixed_prefill_tokens: Optional[int] = None,
        batching_policy: BatchingPolicy = BatchingPolicy.CONTINUOUS,
        ops=None,
        **kwargs,
    ) -> "ContinuousBatchEngine":
        from .factory import default_ops, load_model, make_cache, parse_dtype

        dtype = parse_dtype(dtype)
        ops = ops or default_ops(dtype, device)
        _, model = load_model(model_dir, dtype=dtype, device=ops.device)
        cache = make_cache(model, block_size=block_size, num_blocks=num_blocks, max_requests=max_running_requests)
        runner = ModelRunner(model, cache, ops)
        admission = PagedBlockAdmissionController(cache, max_step_tokens=max_batch_tokens)
        scheduler = RequestScheduler(
            max_running_requests=max_running_requests,
            max_batch_tokens=max_batch_tokens,
            max_mixed_prefill_tokens=max_mixed_prefill_tokens,
            admission_callback=admission.try_admit,
            batching_policy=batching_policy,
        )
        return cls(scheduler=scheduler, runner=runner, admission=admission, **kwargs)

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
        with _trace_range(self.enable_tracing, "scheduler.schedule_step"):
            batch = self.scheduler.schedule_step()
        if batch is None:
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
            with _trace_range(self.enable_tracing, f"model.step:tokens={batch.token_count}"):
                output = self.runner.step(entries)
            chosen = None
            if output.logits is not None:
                chosen = self.sampler.sample(output.logits, params, indices)
        except Exception:
            with _trace_range(self.enable_tracing, "engine.rollback"):
                self.admission.release_admitted(batch.admitted_request_ids)
                self.scheduler.abort_step()
            raise

        with _trace_range(self.enable_tracing, "token.d2h_sync"):
            host_tokens = chosen.cpu().tolist() if chosen is not None else []
        tokens_ready_ns = self._clock_ns()
        generated = {rid: int(tok) for (rid, _), tok in zip(output.rows, host_tokens)}
        with _trace_range(self.enable_tracing, "scheduler.apply_and_release"):
            update = self.scheduler.apply_step_results(generated)
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
