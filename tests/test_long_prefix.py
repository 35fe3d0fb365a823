"""Prompt portions behind thousands of cached tokens, through the step function.

The launch plan of the attention kernels changes with the number of keys before a step's
query tiles: from 2,048 on the wide tiles are chosen earlier, from 4,096 on the keys of few
tiles are cut into runs that a second kernel merges.  A request of some 4,700 tokens is fed in
portions of 512 beside two requests that decode, so that its later portions sit behind both
thresholds; a second request of the same length repeats every step's sizes, so that those steps
are recorded as graphs and replayed.  Compared with the plain implementation, and unrecorded
against recorded bit for bit.
"""

from __future__ import annotations

import pytest
import torch

import plain_qwen2 as plain
from helpers import TINY_A, StepEntry, make_runner, random_tokens, read_weights
from mini_llm_runtime_amd.config import Qwen2Config
from mini_llm_runtime_amd.weights import save_state_dict, write_random_model

pytestmark = pytest.mark.gpu

LONG = 4700
PORTION = 512
BLOCK = 16


def _spying_ops(dtype, tuning):
    from mini_llm_runtime_amd.kernels.ops import HipOps

    class SpyingOps(HipOps):
        """Notes with which tile width and how many key runs the prompt attention was launched."""

        def __init__(self, *args, **kwargs):
            super().__init__(*args, **kwargs)
            self.prefill_launches = []  # (wide, key_runs)

        def _call(self, name, *args, lib=None):
            if name == "mlr_attention_prefill":
                self.prefill_launches.append((int(args[8]), int(args[18])))
            return super()._call(name, *args, lib=lib)

    return SpyingOps(dtype, "cuda", tuning=tuning)


def _run(runner, longs, shorts):
    """Both long requests one after the other, each in portions beside the decoding short ones.
    Returns {(request, position): logits row} and the plan sizes of every step."""
    cache = runner.cache
    got = {}
    plans = []
    seen_plans = runner._plans

    def noting(shape):
        made = seen_plans(shape)
        plans.extend(dict(p.sizes) for p in made)
        return made

    runner._plans = noting
    for rid, toks in shorts.items():
        cache.create_request(rid)
        out = runner.step([StepEntry.of(rid, toks[:3], range(3))])
        for i in range(3):
            got[(rid, i)] = out.logits[i].float().cpu()
    fed_short = {rid: 3 for rid in shorts}
    for rid, toks in longs.items():
        cache.create_request(rid)
        at = 0
        while at < len(toks):
            n = min(PORTION, len(toks) - at)
            wanted = sorted({0, n // 2, n - 1})
            entries = [StepEntry.of(rid, toks[at : at + n], wanted)]
            for sid, stoks in shorts.items():
                if fed_short[sid] < len(stoks):
                    entries.append(StepEntry.of(sid, [stoks[fed_short[sid]]], (0,)))
            out = runner.step(entries)
            rows = out.logits.float().cpu()
            for i, (r, w) in enumerate(out.rows):
                base = at if r == rid else fed_short[r]
                got[(r, base + w)] = rows[i].clone()
            for e in entries[1:]:
                fed_short[e.request_id] += 1
            at += n
            torch.cuda.synchronize()
        cache.release_request(rid)
    for sid in shorts:
        cache.release_request(sid)
    runner._plans = seen_plans
    return got, plans


@pytest.mark.parametrize("wide", [False, True], ids=["tiles64", "tiles128"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_portions_behind_long_prefixes_through_the_step_function(tmp_path, dtype, wide):
    from mini_llm_runtime_amd.kernels.tuning import KernelTuning

    data = dict(TINY_A, max_position_embeddings=8192)
    model_dir = write_random_model(Qwen2Config.from_dict(data), tmp_path / "long", seed=41, storage_dtype="bfloat16")
    cfg, weights = read_weights(model_dir)
    # peaked attention: a far key that is read from a wrong page or left out of a run shows
    weights = {
        n: (t.float() * 6.0).to(t.dtype) if (".q_proj." in n or ".k_proj." in n) else t for n, t in weights.items()
    }
    save_state_dict(model_dir / "model.safetensors", weights)
    vocab = cfg["vocab_size"]
    longs = {f"long{i}": random_tokens(LONG, vocab, 900 + i) for i in range(2)}
    steps_each = -(-LONG // PORTION)
    shorts = {f"short{i}": random_tokens(3 + 2 * steps_each, vocab, 910 + i) for i in range(2)}
    tuning = KernelTuning(wide_attention_groups=1) if wide else KernelTuning()
    pages = -(-LONG // BLOCK) + 2 * (-(-(3 + 2 * steps_each) // BLOCK)) + 2  # pages of the first long request are used again

    results = {}
    for use_graphs in (False, True):
        ops = _spying_ops(dtype, tuning)
        _, _, cache, runner = make_runner(model_dir, ops, block_size=BLOCK, num_blocks=pages, max_requests=4)
        runner.use_graphs = use_graphs
        cache.poison()
        got, plans = _run(runner, longs, shorts)
        cache.check_invariants()
        assert cache.request_ids == ()
        results[use_graphs] = got
        assert {p.get("long_prefix") for p in plans} == {0, 1, 2}, "the portions did not reach both thresholds"
        if dtype == torch.bfloat16:
            assert any(runs > 1 for _, runs in ops.prefill_launches), "no step cut its keys into runs"
            assert any(w == int(wide) and runs > 1 for w, runs in ops.prefill_launches)
            assert {w for w, _ in ops.prefill_launches} == ({1} if wide else {0})
        if use_graphs:
            # (steps of equal sizes share a recording: block tables come in widths of 1,024 tokens)
            levels = {dict(sizes)["long_prefix"] for key in runner._step_graphs for _, sizes in key[5]}
            assert levels == {0, 1, 2}, "steps behind long prefixes were not recorded and replayed"
    plain_rows, recorded = results[False], results[True]
    assert plain_rows.keys() == recorded.keys()
    for key in plain_rows:
        assert torch.equal(plain_rows[key], recorded[key]), f"a recorded step differs from the plain one at {key}"

    everything = {**longs, **shorts}
    worst = (0.0, None)
    for rid, toks in everything.items():
        ref = plain.forward(toks, weights, cfg)
        for (r, pos), row in plain_rows.items():
            if r != rid:
                continue
            row = row.double()
            assert torch.isfinite(row).all(), f"{rid}:{pos} is not finite"
            if dtype == torch.float32:
                assert float((row - ref[pos]).abs().max()) < 2e-4, (rid, pos)
            else:
                worst = max(worst, (float((row - ref[pos]).norm() / ref[pos].norm()), (rid, pos)))
    if dtype == torch.bfloat16:
        # scores of several dozen carry the rounding of queries and keys into the softmax; a key
        # that is missed or taken from a wrong page changes a row by its whole size
        assert worst[0] < 0.2, f"row {worst[1]}: rel L2 error {worst[0]:.3e}"
