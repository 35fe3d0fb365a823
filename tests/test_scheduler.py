"""The scheduler's decisions on the CPU.  The scripted scenarios with requests A-D
follow the reference's tests/test_scheduler.py:14-192 (decode first, FIFO head
blocking, static cohorts, mixed-prefill budget, exact results, abort keeps the step
index); portions of prompts and the page policy are this build's additions."""

from __future__ import annotations

import pytest

from mini_llm_runtime_amd.engine.request import EndReason, Phase, Timeline
from mini_llm_runtime_amd.engine.scheduler import BatchingPolicy, Scheduler


def kinds(plan):
    return [(p.request_id, "prefill" if p.from_prompt else "decode", len(p.tokens)) for p in plan.slices]


def run_step(s, token=7):
    plan = s.plan()
    report = s.complete({rid: token for rid in plan.emitting_ids})
    return plan, report


def test_decode_first_then_fifo_admission():
    s = Scheduler(max_running_requests=3, max_batch_tokens=20, cut_prompts=False)
    s.add("A", [1, 2, 3], max_new_tokens=3)
    s.add("B", [4] * 10, max_new_tokens=2)
    s.add("C", [5] * 9, max_new_tokens=2)
    batch, _ = run_step(s)
    assert kinds(batch) == [("A", "prefill", 3), ("B", "prefill", 10)]  # C (9) does not fit 20 - 13
    assert s.queued_ids == ("C",)
    batch, _ = run_step(s)
    assert kinds(batch) == [("A", "decode", 1), ("B", "decode", 1), ("C", "prefill", 9)]
    assert batch.slices[0].tokens == (7,) and batch.slices[0].offset == 3


def test_head_of_line_blocks_shorter_requests_behind_it():
    s = Scheduler(max_running_requests=4, max_batch_tokens=6, cut_prompts=False)
    s.add("A", [1] * 5, max_new_tokens=2)
    s.add("B", [1] * 6, max_new_tokens=1)
    s.add("C", [1], max_new_tokens=1)
    batch, _ = run_step(s)
    assert kinds(batch) == [("A", "prefill", 5)]  # B does not fit beside A; C must not overtake B
    batch, update = run_step(s)
    assert kinds(batch) == [("A", "decode", 1)] and update.finished == ("A",)
    batch, _ = run_step(s)
    assert kinds(batch) == [("B", "prefill", 6)]


def test_prompt_longer_than_budget_needs_portions():
    s = Scheduler(max_running_requests=2, max_batch_tokens=8, cut_prompts=False)
    with pytest.raises(ValueError, match="max_batch_tokens"):
        s.add("A", [1] * 9, max_new_tokens=1)
    s = Scheduler(max_running_requests=2, max_batch_tokens=8)
    s.add("A", list(range(19)), max_new_tokens=2)
    s.add("B", [1, 2, 3], max_new_tokens=2)
    b1 = s.plan()
    assert kinds(b1) == [("A", "prefill", 8)] and not b1.slices[0].emits
    assert b1.emitting_ids == ()
    s.complete({})
    assert s.request("A").consumed == 8 and s.request("A").generated == ()
    b2, _ = run_step(s)
    assert kinds(b2) == [("A", "prefill", 8)] and b2.slices[0].offset == 8
    b3, _ = run_step(s)  # A's last 3 tokens, and B fills the rest of the budget
    assert kinds(b3) == [("A", "prefill", 3), ("B", "prefill", 3)]
    assert b3.slices[0].tokens == (16, 17, 18) and b3.slices[0].emits
    b4, update = run_step(s)
    assert kinds(b4) == [("A", "decode", 1), ("B", "decode", 1)]
    assert set(update.finished) == {"A", "B"}


def test_a_portion_can_be_a_single_token_beside_decodes():
    s = Scheduler(max_running_requests=3, max_batch_tokens=3)
    s.add("A", [1], max_new_tokens=5)
    s.add("B", [2], max_new_tokens=5)
    run_step(s)
    s.add("C", [9, 8, 7], max_new_tokens=2)
    b, _ = run_step(s)
    assert kinds(b) == [("A", "decode", 1), ("B", "decode", 1), ("C", "prefill", 1)]
    b, _ = run_step(s)
    assert kinds(b) == [("A", "decode", 1), ("B", "decode", 1), ("C", "prefill", 1)] and b.slices[2].offset == 1
    b, _ = run_step(s)
    assert b.slices[2].emits and b.slices[2].tokens == (7,)


def test_mixed_prefill_budget_caps_prompt_tokens_beside_decodes_only():
    s = Scheduler(max_running_requests=4, max_batch_tokens=20, max_mixed_prefill_tokens=4)
    s.add("A", [1] * 10, max_new_tokens=4)
    b, _ = run_step(s)
    assert kinds(b) == [("A", "prefill", 10)]  # nothing is decoding: the cap does not apply
    s.add("B", [2] * 9, max_new_tokens=2)
    b, _ = run_step(s)
    assert kinds(b) == [("A", "decode", 1), ("B", "prefill", 4)]
    b, _ = run_step(s)
    assert kinds(b) == [("A", "decode", 1), ("B", "prefill", 4)]
    b, _ = run_step(s)
    assert kinds(b) == [("A", "decode", 1), ("B", "prefill", 1)] and b.slices[1].emits


def test_static_policy_admits_only_into_an_empty_engine():
    s = Scheduler(max_running_requests=4, max_batch_tokens=32, batching_policy=BatchingPolicy.STATIC)
    s.add("A", [1, 2], max_new_tokens=2)
    s.add("B", [3], max_new_tokens=3)
    b, _ = run_step(s)
    assert kinds(b) == [("A", "prefill", 2), ("B", "prefill", 1)]  # the first cohort may hold several
    s.add("C", [4], max_new_tokens=1)
    b, _ = run_step(s)
    assert kinds(b) == [("A", "decode", 1), ("B", "decode", 1)]  # no refill while the cohort runs
    b, _ = run_step(s)
    assert kinds(b) == [("B", "decode", 1)]
    b, _ = run_step(s)
    assert kinds(b) == [("C", "prefill", 1)]


def test_results_must_match_the_batch_exactly():
    s = Scheduler(max_running_requests=2, max_batch_tokens=8)
    s.add("A", [1], max_new_tokens=2)
    s.add("B", [2], max_new_tokens=2)
    s.plan()
    with pytest.raises(RuntimeError):
        s.plan()  # one outstanding batch at a time
    with pytest.raises(ValueError, match="missing=\\['B'\\]"):
        s.complete({"A": 1})
    with pytest.raises(ValueError, match="extra=\\['Z'\\]"):
        s.complete({"A": 1, "B": 2, "Z": 3})
    with pytest.raises(ValueError):
        s.complete({"A": 1, "B": -2})
    assert s.request("A").generated == ()  # nothing was applied
    s.complete({"A": 1, "B": 2})
    with pytest.raises(RuntimeError):
        s.complete({})


def test_eos_beats_max_tokens_and_finish_reasons():
    s = Scheduler(max_running_requests=2, max_batch_tokens=8)
    s.add("A", [1], max_new_tokens=1, stop_tokens=7)
    s.add("B", [1], max_new_tokens=2, stop_tokens=[3, 4])
    _, update = run_step(s, token=7)
    assert update.finished == ("A",)
    assert s.request("A").end_reason is EndReason.STOP_TOKEN
    assert s.request("A").phase is Phase.DONE
    _, update = run_step(s, token=9)
    assert s.request("B").end_reason is EndReason.LENGTH
    assert s.done_ids == ("A", "B") and not s.busy
    assert s.plan() is None


def test_abort_puts_admitted_requests_back_in_front_and_keeps_the_step_index():
    s = Scheduler(max_running_requests=3, max_batch_tokens=16)
    s.add("A", [1, 2], max_new_tokens=3)
    run_step(s)
    s.add("B", [3], max_new_tokens=1)
    s.add("C", [4], max_new_tokens=1)
    batch = s.plan()
    assert batch.index == 1 and batch.admitted == ("B", "C")
    s.add("D", [5], max_new_tokens=1)  # arrives while the batch is in flight
    s.cancel()
    assert s.queued_ids == ("B", "C", "D") and s.active_ids == ("A",)
    again = s.plan()
    assert again.index == 1 and kinds(again)[:3] == kinds(batch)


def test_admission_callback_false_blocks_the_queue_without_side_effects():
    answers = {"A": True, "B": False, "C": True}
    asked = []

    def admit(request):
        asked.append(request.id)
        return answers[request.id]

    s = Scheduler(max_running_requests=4, max_batch_tokens=16, admit=admit)
    for rid in "ABC":
        s.add(rid, [1], max_new_tokens=2)
    b, _ = run_step(s)
    assert kinds(b) == [("A", "prefill", 1)] and asked == ["A", "B"]  # C is never asked: it is behind B
    assert s.request("B").phase is Phase.QUEUED
    answers["B"] = True
    b, _ = run_step(s)
    assert [k[0] for k in kinds(b)] == ["A", "B", "C"]
    s2 = Scheduler(max_running_requests=1, max_batch_tokens=4, admit=lambda r: False)
    s2.add("X", [1], max_new_tokens=1)
    assert s2.plan() is None and s2.busy  # waits; nothing to run


def test_validation():
    with pytest.raises(ValueError):
        Scheduler(max_running_requests=5, max_batch_tokens=4)
    with pytest.raises(ValueError):
        Scheduler(max_running_requests=1, max_batch_tokens=4, max_mixed_prefill_tokens=0)
    s = Scheduler(max_running_requests=1, max_batch_tokens=4)
    for bad in ([], [1, -1], [True]):
        with pytest.raises(ValueError):
            s.add("x", bad, max_new_tokens=1)
    with pytest.raises(ValueError):
        s.add("", [1], max_new_tokens=1)
    with pytest.raises(ValueError):
        s.add("x", [1], max_new_tokens=0)
    s.add("x", [1], max_new_tokens=1)
    with pytest.raises(ValueError):
        s.add("x", [1], max_new_tokens=1)
    assert s.request("x").cache_tokens == 1  # prompt + max_new - 1


def test_timeline_figures_and_order_of_moments():
    """Definitions of the reference's request metrics (request_metrics.py:20-94): everything counts
    from the arrival, a token's moment is when the host sees it, end-to-end ends at the last
    token and the clean-up after it is a figure of its own; moments never go back in time."""
    t = Timeline()
    with pytest.raises(RuntimeError, match="before it arrives"):
        t.stamp("token", 5)
    t.stamp("arrived", 1_000_000)
    assert t.figures_ms() == {"queue_wait_ms": None, "ttft_ms": None, "median_tpot_ms": None, "e2e_ms": None, "cleanup_ms": None}
    with pytest.raises(RuntimeError, match="without tokens"):
        t.stamp("done", 2_000_000)
    t.stamp("scheduled", 3_000_000)
    t.stamp("scheduled", 4_000_000)  # the step failed and was tried again
    for moment in (9_000_000, 11_000_000, 12_000_000, 16_000_000):
        t.stamp("token", moment)
    with pytest.raises(ValueError, match="back in time"):
        t.stamp("token", 15_000_000)
    with pytest.raises(RuntimeError, match="start its prompt again"):
        t.stamp("scheduled", 17_000_000)
    t.stamp("done", 16_500_000)
    assert t.figures_ms() == {"queue_wait_ms": 2.0, "ttft_ms": 8.0, "median_tpot_ms": 2.0, "e2e_ms": 15.0, "cleanup_ms": 0.5}
    assert t.gaps_ns == (2_000_000, 1_000_000, 4_000_000)
    with pytest.raises(RuntimeError, match="after it is done"):
        t.stamp("token", 17_000_000)
    for bad in (-1, 1.5, True):
        with pytest.raises(ValueError):
            Timeline().stamp("arrived", bad)
