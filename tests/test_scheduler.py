"""The scheduler's decisions on the CPU.  The scripted scenarios with requests A-D
follow the reference's tests/test_scheduler.py:14-192 (decode first, FIFO head
blocking, static cohorts, mixed-prefill budget, exact results, abort keeps the step
index); portions of prompts and the page policy are this build's additions."""

from __future__ import annotations

import pytest

from mini_llm_runtime_amd.engine.scheduler import (
    BatchingPolicy,
    FinishReason,
    RequestScheduler,
    RequestStatus,
)


def kinds(batch):
    return [(i.request_id, i.kind.value, len(i.input_token_ids)) for i in batch.items]


def run_step(s, token=7):
    batch = s.schedule_step()
    update = s.apply_step_results({rid: token for rid in batch.producing_request_ids})
    return batch, update


def test_decode_first_then_fifo_admission():
    s = RequestScheduler(max_running_requests=3, max_batch_tokens=20, chunked_prefill=False)
    s.submit("A", [1, 2, 3], max_new_tokens=3)
    s.submit("B", [4] * 10, max_new_tokens=2)
    s.submit("C", [5] * 9, max_new_tokens=2)
    batch, _ = run_step(s)
    assert kinds(batch) == [("A", "prefill", 3), ("B", "prefill", 10)]  # C (9) does not fit 20 - 13
    assert s.waiting_request_ids == ("C",)
    batch, _ = run_step(s)
    assert kinds(batch) == [("A", "decode", 1), ("B", "decode", 1), ("C", "prefill", 9)]
    assert batch.items[0].input_token_ids == (7,) and batch.items[0].start == 3


def test_head_of_line_blocks_shorter_requests_behind_it():
    s = RequestScheduler(max_running_requests=4, max_batch_tokens=6, chunked_prefill=False)
    s.submit("A", [1] * 5, max_new_tokens=2)
    s.submit("B", [1] * 6, max_new_tokens=1)
    s.submit("C", [1], max_new_tokens=1)
    batch, _ = run_step(s)
    assert kinds(batch) == [("A", "prefill", 5)]  # B does not fit beside A; C must not overtake B
    batch, update = run_step(s)
    assert kinds(batch) == [("A", "decode", 1)] and update.finished_request_ids == ("A",)
    batch, _ = run_step(s)
    assert kinds(batch) == [("B", "prefill", 6)]


def test_prompt_longer_than_budget_needs_portions():
    s = RequestScheduler(max_running_requests=2, max_batch_tokens=8, chunked_prefill=False)
    with pytest.raises(ValueError, match="max_batch_tokens"):
        s.submit("A", [1] * 9, max_new_tokens=1)
    s = RequestScheduler(max_running_requests=2, max_batch_tokens=8)
    s.submit("A", list(range(19)), max_new_tokens=2)
    s.submit("B", [1, 2, 3], max_new_tokens=2)
    b1 = s.schedule_step()
    assert kinds(b1) == [("A", "prefill", 8)] and not b1.items[0].produces_token
    assert b1.producing_request_ids == ()
    s.apply_step_results({})
    assert s.get_request("A").num_computed_tokens == 8 and s.get_request("A").generated_token_ids == ()
    b2, _ = run_step(s)
    assert kinds(b2) == [("A", "prefill", 8)] and b2.items[0].start == 8
    b3, _ = run_step(s)  # A's last 3 tokens, and B fills the rest of the budget
    assert kinds(b3) == [("A", "prefill", 3), ("B", "prefill", 3)]
    assert b3.items[0].input_token_ids == (16, 17, 18) and b3.items[0].produces_token
    b4, update = run_step(s)
    assert kinds(b4) == [("A", "decode", 1), ("B", "decode", 1)]
    assert set(update.finished_request_ids) == {"A", "B"}


def test_a_portion_can_be_a_single_token_beside_decodes():
    s = RequestScheduler(max_running_requests=3, max_batch_tokens=3)
    s.submit("A", [1], max_new_tokens=5)
    s.submit("B", [2], max_new_tokens=5)
    run_step(s)
    s.submit("C", [9, 8, 7], max_new_tokens=2)
    b, _ = run_step(s)
    assert kinds(b) == [("A", "decode", 1), ("B", "decode", 1), ("C", "prefill", 1)]
    b, _ = run_step(s)
    assert kinds(b) == [("A", "decode", 1), ("B", "decode", 1), ("C", "prefill", 1)] and b.items[2].start == 1
    b, _ = run_step(s)
    assert b.items[2].produces_token and b.items[2].input_token_ids == (7,)


def test_mixed_prefill_budget_caps_prompt_tokens_beside_decodes_only():
    s = RequestScheduler(max_running_requests=4, max_batch_tokens=20, max_mixed_prefill_tokens=4)
    s.submit("A", [1] * 10, max_new_tokens=4)
    b, _ = run_step(s)
    assert kinds(b) == [("A", "prefill", 10)]  # nothing is decoding: the cap does not apply
    s.submit("B", [2] * 9, max_new_tokens=2)
    b, _ = run_step(s)
    assert kinds(b) == [("A", "decode", 1), ("B", "prefill", 4)]
    b, _ = run_step(s)
    assert kinds(b) == [("A", "decode", 1), ("B", "prefill", 4)]
    b, _ = run_step(s)
    assert kinds(b) == [("A", "decode", 1), ("B", "prefill", 1)] and b.items[1].produces_token


def test_static_policy_admits_only_into_an_empty_engine():
    s = RequestScheduler(max_running_requests=4, max_batch_tokens=32, batching_policy=BatchingPolicy.STATIC)
    s.submit("A", [1, 2], max_new_tokens=2)
    s.submit("B", [3], max_new_tokens=3)
    b, _ = run_step(s)
    assert kinds(b) == [("A", "prefill", 2), ("B", "prefill", 1)]  # the first cohort may hold several
    s.submit("C", [4], max_new_tokens=1)
    b, _ = run_step(s)
    assert kinds(b) == [("A", "decode", 1), ("B", "decode", 1)]  # no refill while the cohort runs
    b, _ = run_step(s)
    assert kinds(b) == [("B", "decode", 1)]
    b, _ = run_step(s)
    assert kinds(b) == [("C", "prefill", 1)]


def test_results_must_match_the_batch_exactly():
    s = RequestScheduler(max_running_requests=2, max_batch_tokens=8)
    s.submit("A", [1], max_new_tokens=2)
    s.submit("B", [2], max_new_tokens=2)
    s.schedule_step()
    with pytest.raises(RuntimeError):
        s.schedule_step()  # one outstanding batch at a time
    with pytest.raises(ValueError, match="missing=\\['B'\\]"):
        s.apply_step_results({"A": 1})
    with pytest.raises(ValueError, match="extra=\\['Z'\\]"):
        s.apply_step_results({"A": 1, "B": 2, "Z": 3})
    with pytest.raises(ValueError):
        s.apply_step_results({"A": 1, "B": -2})
    assert s.get_request("A").generated_token_ids == ()  # nothing was applied
    s.apply_step_results({"A": 1, "B": 2})
    with pytest.raises(RuntimeError):
        s.apply_step_results({})


def test_eos_beats_max_tokens_and_finish_reasons():
    s = RequestScheduler(max_running_requests=2, max_batch_tokens=8)
    s.submit("A", [1], max_new_tokens=1, eos_token_ids=7)
    s.submit("B", [1], max_new_tokens=2, eos_token_ids=[3, 4])
    _, update = run_step(s, token=7)
    assert update.finished_request_ids == ("A",)
    assert s.get_request("A").finish_reason is FinishReason.EOS
    assert s.get_request("A").status is RequestStatus.FINISHED
    _, update = run_step(s, token=9)
    assert s.get_request("B").finish_reason is FinishReason.MAX_TOKENS
    assert s.finished_request_ids == ("A", "B") and not s.has_unfinished_requests
    assert s.schedule_step() is None


def test_abort_puts_admitted_requests_back_in_front_and_keeps_the_step_index():
    s = RequestScheduler(max_running_requests=3, max_batch_tokens=16)
    s.submit("A", [1, 2], max_new_tokens=3)
    run_step(s)
    s.submit("B", [3], max_new_tokens=1)
    s.submit("C", [4], max_new_tokens=1)
    batch = s.schedule_step()
    assert batch.step_index == 1 and batch.admitted_request_ids == ("B", "C")
    s.submit("D", [5], max_new_tokens=1)  # arrives while the batch is in flight
    s.abort_step()
    assert s.waiting_request_ids == ("B", "C", "D") and s.running_request_ids == ("A",)
    again = s.schedule_step()
    assert again.step_index == 1 and kinds(again)[:3] == kinds(batch)


def test_admission_callback_false_blocks_the_queue_without_side_effects():
    answers = {"A": True, "B": False, "C": True}
    asked = []

    def admit(request):
        asked.append(request.request_id)
        return answers[request.request_id]

    s = RequestScheduler(max_running_requests=4, max_batch_tokens=16, admission_callback=admit)
    for rid in "ABC":
        s.submit(rid, [1], max_new_tokens=2)
    b, _ = run_step(s)
    assert kinds(b) == [("A", "prefill", 1)] and asked == ["A", "B"]  # C is never asked: it is behind B
    assert s.get_request("B").status is RequestStatus.WAITING
    answers["B"] = True
    b, _ = run_step(s)
    assert [k[0] for k in kinds(b)] == ["A", "B", "C"]
    s2 = RequestScheduler(max_running_requests=1, max_batch_tokens=4, admission_callback=lambda r: False)
    s2.submit("X", [1], max_new_tokens=1)
    assert s2.schedule_step() is None and s2.has_unfinished_requests  # waits; nothing to run


def test_validation():
    with pytest.raises(ValueError):
        RequestScheduler(max_running_requests=5, max_batch_tokens=4)
    with pytest.raises(ValueError):
        RequestScheduler(max_running_requests=1, max_batch_tokens=4, max_mixed_prefill_tokens=0)
    s = RequestScheduler(max_running_requests=1, max_batch_tokens=4)
    for bad in ([], [1, -1], [True]):
        with pytest.raises(ValueError):
            s.submit("x", bad, max_new_tokens=1)
    with pytest.raises(ValueError):
        s.submit("", [1], max_new_tokens=1)
    with pytest.raises(ValueError):
        s.submit("x", [1], max_new_tokens=0)
    s.submit("x", [1], max_new_tokens=1)
    with pytest.raises(ValueError):
        s.submit("x", [1], max_new_tokens=1)
    assert s.get_request("x").max_cache_tokens == 1  # prompt + max_new - 1
