"""Generation through the entry points: single-request greedy generation, the
continuous-batching engine with late arrivals, page pressure, temperature sampling,
and rollback of a failed step.  On the CPU with the torch stand-in for the kernels,
on the GPU (`-m gpu`) with the HIP kernels in 32-bit and bfloat16."""

from __future__ import annotations

import pytest
import torch

import mini_llm_runtime_amd as mlr
import plain_qwen2 as plain
from helpers import BLOCK_SIZE, TINY, make_model_dir, random_tokens, read_weights
from kernel_doubles import TorchOps
from mini_llm_runtime_amd.engine import (
    BatchingPolicy,
    ContinuousBatchEngine,
    ModelRunner,
    PageAdmission,
    Scheduler,
)

CASES = [
    pytest.param("double", torch.float32, id="double-f32"),
    pytest.param("hip", torch.float32, id="hip-f32", marks=pytest.mark.gpu),
    pytest.param("hip", torch.bfloat16, id="hip-bf16", marks=pytest.mark.gpu),
]


def _ops(backend, dtype):
    if backend == "double":
        return TorchOps(dtype, "cpu")
    from mini_llm_runtime_amd.kernels.ops import HipOps

    return HipOps(dtype, "cuda")


def _engine(model_dir, ops, *, block_size, num_blocks, max_running=4, max_batch_tokens=32, **kw):
    return ContinuousBatchEngine.from_model_dir(
        model_dir, dtype=ops.dtype, ops=ops, block_size=block_size, num_blocks=num_blocks,
        max_running_requests=max_running, max_batch_tokens=max_batch_tokens, **kw,
    )


def _check_greedy(tokens, prompt, weights, cfg, dtype):
    """Exact in 32-bit; in bfloat16 a difference is allowed only where the plain
    implementation's two best logits are nearly tied."""
    seq = list(prompt)
    for i, tok in enumerate(tokens):
        logits = plain.forward(seq, weights, cfg)[-1]
        best = int(torch.argmax(logits))
        if tok != best:
            assert dtype == torch.bfloat16, f"token {i}: {tok} != {best}"
            top = torch.topk(logits, 2).values
            assert float(top[0] - logits[tok]) < 2e-2 * float(logits.abs().max()), f"token {i} differs on a clear margin"
            return
        seq.append(tok)


@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("which", ["A", "B"])
def test_greedy_generate_matches_recompute_everything(tmp_path, which, backend, dtype):
    """Cached generation == the plain recompute-everything loop (reference tests/test_generation.py:14-52)."""
    d = make_model_dir(tmp_path, which, seed=21)
    cfg, w = read_weights(d)
    ops = _ops(backend, dtype)
    _, model = mlr.load_model(d, dtype=dtype, device=ops.device)
    cache = mlr.make_cache(model, block_size=3, num_blocks=20, max_requests=2)  # block size 3: growth across pages
    runner = ModelRunner(model, cache, ops)
    prompt = random_tokens(17, cfg["vocab_size"], 5)
    out = mlr.greedy_generate(runner, prompt, max_new_tokens=8, return_step_logits=True)
    assert len(out.generated_token_ids) == 8 and out.decode_steps == 7 and out.prefill_tokens == 17
    assert out.cache_length == 17 + 8 - 1  # the last token is never fed back
    _check_greedy(out.generated_token_ids, prompt, w, cfg, dtype)
    if dtype == torch.float32:
        seq = list(prompt)
        for i, tok in enumerate(out.generated_token_ids):
            ref = plain.forward(seq, w, cfg)[-1]
            assert float((out.step_logits[i].double().cpu() - ref).abs().max()) < 1e-4
            seq.append(tok)
    assert cache.request_ids == () and cache.groups[0].allocator.free_count == 20
    # EOS stops without a further step (reference tests/test_generation.py:54-71)
    eos = out.generated_token_ids[2]
    first = out.generated_token_ids.index(eos)
    stopped = mlr.greedy_generate(runner, prompt, max_new_tokens=8, eos_token_ids=eos)
    assert stopped.stopped_by_eos and stopped.generated_token_ids == out.generated_token_ids[: first + 1]
    assert stopped.decode_steps == first
    with pytest.raises(RuntimeError, match="free pages"):
        mlr.greedy_generate(runner, prompt, max_new_tokens=60)
    with pytest.raises(ValueError):
        mlr.greedy_generate(runner, prompt, max_new_tokens=8, eos_token_ids=cfg["vocab_size"])


@pytest.mark.parametrize("backend,dtype", CASES)
def test_continuous_batching_with_late_arrivals(tmp_path, backend, dtype):
    """Tiny B workload: prompts 1/9/24/40/63 arriving at steps 0/0/2/3/5, 12 new tokens each."""
    d = make_model_dir(tmp_path, "B", seed=22)
    cfg, w = read_weights(d)
    ops = _ops(backend, dtype)
    engine = _engine(d, ops, block_size=BLOCK_SIZE["B"], num_blocks=40, max_running=4, max_batch_tokens=32)
    lengths = {"r0": 1, "r1": 9, "r2": 24, "r3": 40, "r4": 63}
    arrivals = {"r0": 0, "r1": 0, "r2": 2, "r3": 3, "r4": 5}
    prompts = {rid: random_tokens(n, cfg["vocab_size"], 40 + i) for i, (rid, n) in enumerate(lengths.items())}
    step = 0
    saw_mixed = saw_portion = False
    reused: set[int] = set()
    freed: set[int] = set()
    while step < 200:
        for rid, at in arrivals.items():
            if at == step:
                engine.submit(rid, prompts[rid], max_new_tokens=12)
        if not engine.scheduler.busy and step > max(arrivals.values()):
            break
        result = engine.step()
        step += 1
        if result is None:
            continue
        b = result.plan
        saw_mixed |= bool(b.decode_ids) and bool(b.prompt_ids)
        saw_portion |= any(not p.emits for p in b.slices)
        held = {p for rid in engine.manager.request_ids for p in engine.manager.get_request(rid).live_blocks(0)}
        reused |= held & freed
        for _, blocks in result.released_blocks:
            freed |= set(blocks[0])
        engine.manager.check_invariants()
    assert saw_mixed and saw_portion and reused, "the workload must mix, cut prompts and use pages again"
    for rid, prompt in prompts.items():
        tokens = engine.request(rid).generated
        assert len(tokens) == 12
        _check_greedy(tokens, prompt, w, cfg, dtype)
    assert engine.manager.request_ids == () and engine.admission.promises == ()
    assert engine.manager.groups[0].allocator.free_count == 40
    line = engine.request("r4").timeline
    assert line.ttft_ns > 0 and len(line.gaps_ns) == 11 and line.e2e_ns >= line.ttft_ns and line.cleanup_ns >= 0
    m = engine.times("r4")
    assert m.tokens == 12 and m.ttft_ms == line.ttft_ns / 1e6 and m.queue_wait_ms >= 0
    assert len(engine.all_times()) == 5


@pytest.mark.parametrize("backend,dtype", CASES[:2])
def test_temperature_sampling_is_reproducible_and_independent_of_the_batch(tmp_path, backend, dtype):
    d = make_model_dir(tmp_path, "B", seed=23)
    cfg, _ = read_weights(d)
    ops = _ops(backend, dtype)
    prompts = [random_tokens(n, cfg["vocab_size"], 60 + n) for n in (5, 19, 33)]

    def run(which, max_running):
        engine = _engine(d, ops, block_size=8, num_blocks=64, max_running=max_running, max_batch_tokens=16)
        for i in which:
            engine.submit(f"s{i}", prompts[i], max_new_tokens=10, temperature=0.8, seed=1000 + i)
        engine.run_until_done()
        return {i: engine.request(f"s{i}").generated for i in which}

    together = run([0, 1, 2], 3)
    again = run([0, 1, 2], 3)
    assert together == again
    alone = {}
    for i in range(3):
        alone.update(run([i], 1))
    assert alone == together, "sampled tokens changed with the batch composition"
    greedy = _engine(d, ops, block_size=8, num_blocks=64).generate(prompts, max_new_tokens=10)
    assert [list(together[i]) for i in range(3)] != greedy, "temperature 0.8 should not reproduce greedy everywhere"


@pytest.mark.parametrize("backend,dtype", CASES[:2])
def test_pages_run_out_requests_wait_then_enter(tmp_path, backend, dtype):
    """Admission by lifetime pages: a request that does not fit waits at the head; one that can never fit raises."""
    d = make_model_dir(tmp_path, "A", seed=24)
    cfg, w = read_weights(d)
    ops = _ops(backend, dtype)
    engine = _engine(d, ops, block_size=4, num_blocks=6, max_running=3, max_batch_tokens=16)
    p1, p2 = random_tokens(10, cfg["vocab_size"], 1), random_tokens(9, cfg["vocab_size"], 2)
    engine.submit("big", p1, max_new_tokens=4)  # 13 tokens -> 4 pages
    engine.submit("late", p2, max_new_tokens=3)  # 11 tokens -> 3 pages: does not fit beside "big"
    first = engine.step()
    assert first.plan.prompt_ids == ("big",) and engine.scheduler.queued_ids == ("late",)
    order = []
    while engine.scheduler.busy:
        r = engine.step()
        order.append((r.plan.prompt_ids, r.report.finished))
    assert any(p == ("late",) for p, _ in order)
    done_big = next(i for i, (_, f) in enumerate(order) if "big" in f)
    enter_late = next(i for i, (p, _) in enumerate(order) if p == ("late",))
    assert enter_late == done_big + 1  # the step after the pages came back
    _check_greedy(engine.request("late").generated, p2, w, cfg, dtype)
    # 27 tokens -> 7 pages > 6: refused when it is submitted, so it never blocks the queue
    with pytest.raises(ValueError, match="never"):
        engine.submit("never", random_tokens(20, cfg["vocab_size"], 3), max_new_tokens=8)
    assert "never" not in engine.scheduler.queued_ids and engine.step() is None


@pytest.mark.parametrize("backend,dtype", CASES[:2])
def test_failed_step_rolls_back_and_can_be_retried(tmp_path, backend, dtype):
    """A failure inside the model leaves scheduler and cache as before the step; the retry has the
    same step index and the same outcome (reference tests/test_engine.py:329-389)."""
    d = make_model_dir(tmp_path, "A", seed=25)
    cfg, w = read_weights(d)
    ops = _ops(backend, dtype)
    engine = _engine(d, ops, block_size=4, num_blocks=32, max_running=3, max_batch_tokens=32)
    pa, pc = random_tokens(7, cfg["vocab_size"], 1), random_tokens(5, cfg["vocab_size"], 2)
    engine.submit("A", pa, max_new_tokens=4)
    engine.step()
    engine.submit("C", pc, max_new_tokens=3)
    before = (engine.manager.get_request("A").num_tokens, engine.manager.groups[0].allocator.free_count)
    engine.runner.fail_next_step = RuntimeError("injected")
    with pytest.raises(RuntimeError, match="injected"):
        engine.step()
    assert engine.scheduler.queued_ids == ("C",) and engine.scheduler.active_ids == ("A",)
    assert not engine.manager.has_request("C") and engine.admission.promises[0].request_id == "A"
    assert (engine.manager.get_request("A").num_tokens, engine.manager.groups[0].allocator.free_count) == before
    engine.manager.check_invariants()
    retry = engine.step()
    assert retry.plan.index == 1
    assert retry.plan.decode_ids == ("A",) and retry.plan.prompt_ids == ("C",)
    engine.run_until_done()
    _check_greedy(engine.request("A").generated, pa, w, cfg, dtype)
    _check_greedy(engine.request("C").generated, pc, w, cfg, dtype)


def test_a_failure_after_the_cache_counted_the_step_stops_the_engine(tmp_path):
    """When choosing the tokens fails, the step's tokens are already cached: cancelling the plan
    would feed them again behind themselves.  The engine refuses to go on instead, and leaves
    the scheduler's plan outstanding rather than rolled back."""
    from mini_llm_runtime_amd.engine.engine import EngineBrokenError

    d = make_model_dir(tmp_path, "A", seed=26)
    cfg, _ = read_weights(d)
    engine = _engine(d, _ops("double", torch.float32), block_size=4, num_blocks=32, max_running=3)
    engine.submit("A", random_tokens(7, cfg["vocab_size"], 1), max_new_tokens=4)
    engine.step()
    cached = engine.manager.get_request("A").num_tokens

    def broken_sampler(*args, **kwargs):
        raise RuntimeError("no tokens today")

    engine.sampler.sample = broken_sampler
    with pytest.raises(EngineBrokenError, match="no tokens today"):
        engine.step()
    assert engine.manager.get_request("A").num_tokens == cached + 1  # the step counted
    assert engine.scheduler.active_ids == ("A",)  # and nothing was rolled back behind it
    with pytest.raises(EngineBrokenError, match="cannot go on"):
        engine.step()


def test_a_plan_that_disagrees_with_the_cache_is_refused(tmp_path):
    """Every slice must go on where its request's cache ends."""
    d = make_model_dir(tmp_path, "A", seed=27)
    cfg, _ = read_weights(d)
    engine = _engine(d, _ops("double", torch.float32), block_size=4, num_blocks=32, max_running=3, lookahead=False)
    engine.submit("A", random_tokens(9, cfg["vocab_size"], 1), max_new_tokens=4)
    engine.step()
    # a step behind the scheduler's back: the cache is now one token ahead of the plan to come
    engine.runner.step([mlr.StepEntry.of("A", [1])])
    with pytest.raises(RuntimeError, match="the cache holds"):
        engine.step()
    # the refused step was rolled back like any failed one
    assert engine.scheduler.active_ids == ("A",) and not engine.manager.step_in_flight


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_decoding_one_step_ahead_changes_nothing_but_the_waiting(tmp_path, dtype):
    """The engine launches the next decode step before it has seen the last one's tokens.  With
    requests that end on an end-of-sequence token at different times, late arrivals and few
    pages, every request's tokens, every batch and every released page must be those of the
    plain loop; launches are both confirmed and abandoned on the way; no page is lost."""
    d = make_model_dir(tmp_path, "B", seed=29)
    cfg, w = read_weights(d)
    from mini_llm_runtime_amd.kernels.ops import HipOps

    lengths = {"r0": 3, "r1": 9, "r2": 24, "r3": 17, "r4": 30, "r5": 2}
    arrivals = {"r0": 0, "r1": 0, "r2": 1, "r3": 9, "r4": 9, "r5": 30}
    prompts = {rid: random_tokens(n, cfg["vocab_size"], 60 + i) for i, (rid, n) in enumerate(lengths.items())}

    def run(lookahead, eos):
        engine = _engine(d, HipOps(dtype, "cuda"), block_size=BLOCK_SIZE["B"], num_blocks=30, max_running=3,
                         max_batch_tokens=32, lookahead=lookahead)
        trace = []
        step = 0
        while step < 300:
            for rid, at in arrivals.items():
                if at == step:
                    engine.submit(rid, prompts[rid], max_new_tokens=24, temperature=0.7 if rid == "r1" else 0.0,
                                  seed=5, eos_token_ids=eos)
            if not engine.scheduler.busy and step > max(arrivals.values()):
                break
            result = engine.step()
            step += 1
            if result is not None:
                trace.append((tuple((p.request_id, p.from_prompt, p.tokens) for p in result.plan.slices),
                              result.report.emitted, result.report.finished, result.released_blocks))
        assert engine.lookahead_error is None
        assert engine.manager.request_ids == () and engine.admission.promises == ()
        assert not engine.manager.step_in_flight
        engine.manager.check_invariants()
        assert engine.manager.groups[0].allocator.free_count == 30
        tokens = {rid: engine.request(rid).generated for rid in prompts}
        return tokens, trace, engine

    plain_tokens, _, _ = run(False, None)
    # end-of-sequence tokens taken from what the requests really generate, so that they end at
    # different steps, some of them while a launch for the next step is out
    eos = {plain_tokens["r0"][5], plain_tokens["r2"][11], plain_tokens["r4"][3]}
    want_tokens, want_trace, off = run(False, eos)
    got_tokens, got_trace, on = run(True, eos)
    assert off.lookahead_hits == 0 and off.lookahead_misses == 0
    assert on.lookahead_hits > 5 and on.lookahead_misses > 0
    assert got_tokens == want_tokens
    assert got_trace == want_trace
    assert any(len(t) < 24 for t in got_tokens.values()), "no request ended on an end-of-sequence token"


def test_static_policy_does_not_refill(tmp_path):
    d = make_model_dir(tmp_path, "A", seed=26)
    cfg, _ = read_weights(d)
    engine = _engine(d, TorchOps(torch.float32), block_size=4, num_blocks=32, batching_policy=BatchingPolicy.STATIC)
    engine.submit("A", [1, 2, 3], max_new_tokens=3)
    engine.step()
    engine.submit("B", [4, 5], max_new_tokens=2)
    r = engine.step()
    assert r.plan.prompt_ids == () and r.plan.decode_ids == ("A",)


def test_engine_checks_its_wiring(tmp_path):
    d = make_model_dir(tmp_path, "A", seed=27)
    ops = TorchOps(torch.float32)
    _, model = mlr.load_model(d, dtype=torch.float32, device="cpu")
    cache = mlr.make_cache(model, block_size=4, num_blocks=8, max_requests=2)
    other = mlr.make_cache(model, block_size=4, num_blocks=8, max_requests=2)
    runner = ModelRunner(model, cache, ops)
    sched = Scheduler(max_running_requests=2, max_batch_tokens=8)
    with pytest.raises(ValueError, match="share one cache"):
        ContinuousBatchEngine(scheduler=sched, runner=runner, admission=PageAdmission(other, max_step_tokens=8))
    big = Scheduler(max_running_requests=3, max_batch_tokens=8)
    with pytest.raises(ValueError, match="slots"):
        ContinuousBatchEngine(scheduler=big, runner=runner, admission=PageAdmission(cache, max_step_tokens=8))
    engine = ContinuousBatchEngine(scheduler=sched, runner=runner, admission=PageAdmission(cache, max_step_tokens=8))
    with pytest.raises(ValueError, match="vocabulary"):
        engine.submit("x", [TINY["A"]["vocab_size"]], max_new_tokens=1)
    with pytest.raises(ValueError, match="max_position"):
        engine.submit("x", [1] * 500, max_new_tokens=20)
