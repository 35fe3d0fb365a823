"""The step function against the plain implementation under every way of cutting
and batching: whole, bulk + one by one, changing portions, and mixed with pages
that are used again.  Runs with the torch stand-in for the kernels on the CPU and
with the HIP kernels on the GPU (`-m gpu`), in 32-bit and in bfloat16.
"""

from __future__ import annotations

import pytest
import torch

import mini_llm_runtime_amd.models  # noqa: F401
import plain_qwen2 as plain
import schedules
from helpers import BLOCK_SIZE, TINY, StepEntry, make_model_dir, make_runner, random_tokens, read_weights
from kernel_doubles import TorchOps

LENGTHS = {
    "A": (5, 17, 33, 70, 41, 52), "B": (1, 9, 24, 40, 63, 37), "C": (3, 65, 34, 97, 40, 51), "D": (2, 19, 35, 66, 45, 50),
    "E": (1, 9, 24, 40, 63, 44),
}

# float32: the engine and the plain implementation (float64) differ by float32
# rounding only.  bfloat16: activations between kernels are rounded to 8 bits of
# mantissa (2^-9 relative per rounding); the error is judged relative to the size
# of the logits.
FP32_MAX_ABS = 1e-4
BF16_ROW_REL_L2 = 5e-2  # of any single row
BF16_REL_L2 = 2e-2


def _ops(backend: str, dtype: torch.dtype):
    if backend == "double":
        return TorchOps(dtype, "cpu")
    from mini_llm_runtime_amd.kernels.ops import HipOps

    return HipOps(dtype, "cuda")


def _sharpen(tensors: dict[str, torch.Tensor], factor: float) -> dict[str, torch.Tensor]:
    """Scale the query and key projections so that attention is peaked: with small
    random weights every key gets nearly the same weight, which would hide a key
    that is read from the wrong place."""
    out = {}
    for name, t in tensors.items():
        if ".q_proj." in name or ".k_proj." in name:
            t = (t.float() * factor).to(t.dtype)
        out[name] = t
    return out


def _setup(tmp_path, which: str, backend: str, dtype: torch.dtype, steps, sharp: float = 0.0):
    from mini_llm_runtime_amd.weights import save_state_dict

    model_dir = make_model_dir(tmp_path, which, seed=11)
    cfg, weights = read_weights(model_dir)
    if sharp:
        weights = _sharpen(weights, sharp)
        save_state_dict(model_dir / "model.safetensors", weights)
    bs = BLOCK_SIZE[which]
    ops = _ops(backend, dtype)
    _, _, cache, runner = make_runner(
        model_dir, ops, block_size=bs, num_blocks=schedules.pages_needed(steps, bs), max_requests=4
    )
    cache.poison()
    return cfg, weights, cache, runner


def _requests(which: str) -> dict[str, list[int]]:
    vocab = TINY[which]["vocab_size"]
    return {f"r{i}": random_tokens(n, vocab, 100 + i) for i, n in enumerate(LENGTHS[which])}


def _compare(got, requests, weights, cfg, dtype, row_bound=None):
    assert got, "no logits came back"
    worst_abs = 0.0
    worst_row = (0.0, None)
    num = 0.0
    den = 0.0
    for rid, toks in requests.items():
        ref = plain.forward(toks, weights, cfg)
        for pos in range(len(toks)):
            row = got[(rid, pos)].double()
            assert torch.isfinite(row).all(), f"{rid}:{pos} is not finite"
            diff = row - ref[pos]
            worst_abs = max(worst_abs, float(diff.abs().max()))
            row_num, row_den = float((diff**2).sum()), float((ref[pos] ** 2).sum())
            worst_row = max(worst_row, ((row_num / row_den) ** 0.5, (rid, pos)))
            num += row_num
            den += row_den
    rel = (num / den) ** 0.5
    if dtype == torch.float32:
        assert worst_abs < FP32_MAX_ABS, f"max abs error {worst_abs:.3e}, rel L2 {rel:.3e}"
    else:
        # all rows together, and every single row: one wrong position among hundreds must not
        # hide in the aggregate
        assert rel < BF16_REL_L2, f"rel L2 error {rel:.3e}, max abs {worst_abs:.3e}"
        assert worst_row[0] < (row_bound or BF16_ROW_REL_L2), f"row {worst_row[1]}: rel L2 error {worst_row[0]:.3e}"


FAMILIES = {
    "whole": schedules.whole,
    "bulk_then_tail": schedules.bulk_then_tail,
    "portions": schedules.portions,
    "mixed": schedules.mixed,
}

CASES = [
    pytest.param("double", torch.float32, id="double-f32"),
    pytest.param("hip", torch.float32, id="hip-f32", marks=pytest.mark.gpu),
    pytest.param("hip", torch.bfloat16, id="hip-bf16", marks=pytest.mark.gpu),
]


@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E"])
def test_schedule_matches_plain(tmp_path, which, family, backend, dtype):
    requests = _requests(which)
    steps = FAMILIES[family](requests)
    if family == "mixed":
        assert schedules.most_live(steps) == 4
        total = sum(schedules.blocks_for(len(t), BLOCK_SIZE[which]) for t in requests.values())
        assert schedules.pages_needed(steps, BLOCK_SIZE[which]) < total, "pages would not be used again"
    cfg, weights, cache, runner = _setup(tmp_path, which, backend, dtype, steps)
    got = schedules.run_schedule(runner, cache, steps)
    _compare(got, requests, weights, cfg, dtype)
    cache.check_invariants()
    assert cache.request_ids == ()
    assert all(g.allocator.free_count == g.num_blocks for g in cache.groups)


@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E"])
def test_peaked_attention_mixed(tmp_path, which, backend, dtype):
    """Same as the mixed family, with query/key projections scaled up so that single
    keys dominate: a key read from a wrong slot or page changes the logits visibly."""
    requests = _requests(which)
    steps = schedules.mixed(requests, seed=5)
    # The spread of the scores grows with factor^2 * width (a query or key entry sums `width`
    # products), and with it what the bfloat16 rounding of queries and keys (2^-9 of a score) does
    # to the softmax, whichever attention kernel runs: at 12 the 96- and 100-wide models sit just
    # under the aggregate bound (1.98e-2 of 2e-2), the 128-wide one above it (3.2e-2).  It gets the
    # spread that the 64-wide model has at 12.
    hidden = TINY[which]["hidden_size"]
    sharp = 12.0 if hidden <= 100 else 12.0 * (64 / hidden) ** 0.5
    cfg, weights, cache, runner = _setup(tmp_path, which, backend, dtype, steps, sharp=sharp)
    got = schedules.run_schedule(runner, cache, steps)
    # Scores this large carry the bfloat16 rounding of q and k (2^-9 of a score of several
    # dozen) into the softmax, so a single row may be off by more than elsewhere; a key taken
    # from a wrong slot changes a row by its whole size (rel L2 near 1).
    _compare(got, requests, weights, cfg, dtype, row_bound=0.2)


@pytest.mark.gpu
@pytest.mark.parametrize("family", ["whole", "portions", "mixed"])
@pytest.mark.parametrize("which", ["A", "B"])
def test_wide_attention_tiles_through_the_step_function(tmp_path, which, family):
    """Prompts of several hundred tokens with the prompt kernel's 128-query tiles forced (these
    few tiles would not choose them): whole, in portions of changing size behind a cached prefix,
    and mixed with decoded tokens of other requests, against the plain implementation."""
    from mini_llm_runtime_amd.kernels.ops import HipOps
    from mini_llm_runtime_amd.kernels.tuning import KernelTuning

    vocab = TINY[which]["vocab_size"]
    requests = {f"w{i}": random_tokens(n, vocab, 300 + i) for i, n in enumerate((150, 290, 133, 260))}
    steps = FAMILIES[family](requests)
    model_dir = make_model_dir(tmp_path, which, seed=13)
    cfg, weights = read_weights(model_dir)
    bs = BLOCK_SIZE[which]
    ops = HipOps(torch.bfloat16, "cuda", tuning=KernelTuning(wide_attention_groups=1))
    _, _, cache, runner = make_runner(model_dir, ops, block_size=bs, num_blocks=schedules.pages_needed(steps, bs), max_requests=4)
    cache.poison()
    got = schedules.run_schedule(runner, cache, steps)
    _compare(got, requests, weights, cfg, torch.bfloat16)
    cache.check_invariants()


@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("which", ["A", "B", "C", "D"])
def test_schedules_agree_with_each_other(tmp_path, which, backend, dtype):
    """The families agree with each other: in 32-bit far below the plain-implementation
    bound; in bfloat16 every single row within what the different kernels of prompt portions
    and single tokens round differently."""
    requests = _requests(which)
    results = []
    for family in FAMILIES.values():
        steps = family(requests)
        _, _, cache, runner = _setup(tmp_path, which, backend, dtype, steps)
        results.append(schedules.run_schedule(runner, cache, steps))
    for other in results[1:]:
        for key, row in results[0].items():
            if dtype == torch.float32:
                assert torch.allclose(row, other[key], atol=2e-5, rtol=0), key
            else:
                rel = float((row - other[key]).norm() / row.norm())
                assert rel < BF16_ROW_REL_L2, (key, rel)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_long_decoding_graph_replays_match_eager(tmp_path, dtype):
    """Decode steps replay a captured HIP graph.  Every replay, with eager steps (portions of a
    further prompt) and synchronisations between the replays, must give exactly what the same
    step gives when its kernels are launched one by one; both follow the plain implementation
    over 100 decoded tokens, across page edges and a change of the graph's batch size."""
    from mini_llm_runtime_amd.kernels.ops import HipOps

    which = "B"
    model_dir = make_model_dir(tmp_path, which, seed=12)
    cfg, weights = read_weights(model_dir)
    vocab = cfg["vocab_size"]
    requests = {f"d{i}": random_tokens(n, vocab, 500 + i) for i, n in enumerate((130, 117, 141))}
    extra = random_tokens(90, vocab, 600)
    ops = HipOps(dtype, "cuda")
    results = []
    for use_graphs in (True, False):
        config, model, cache, runner = make_runner(model_dir, ops, block_size=8, num_blocks=80, max_requests=4)
        runner.use_graphs = use_graphs
        runner.max_decode_graphs = 2  # three batch sizes follow: the graph used longest ago has to go
        cache.poison()
        got = {}
        for rid, toks in requests.items():
            cache.create_request(rid)
            out = runner.step([StepEntry.of(rid, toks[:30], range(30))])
            for i in range(30):
                got[(rid, i)] = out.logits[i].float().cpu()
        cache.create_request("x")
        fed_x = 0
        for step in range(30, 141):
            live = [rid for rid, toks in requests.items() if step < len(toks)]
            out = runner.step([StepEntry.of(rid, [requests[rid][step]], (0,)) for rid in live])
            rows = out.logits.float().cpu()
            for i, rid in enumerate(live):
                got[(rid, step)] = rows[i].clone()
            if step % 7 == 0 and fed_x < len(extra):  # eager work between the replays
                n = min(5, len(extra) - fed_x)
                out = runner.step([StepEntry.of("x", extra[fed_x : fed_x + n], range(n))])
                for i in range(n):
                    got[("x", fed_x + i)] = out.logits[i].float().cpu()
                fed_x += n
        if use_graphs:
            assert len(runner._graphs) == 2, "the decode steps did not go through captured graphs, or too many were kept"
        results.append(got)
    graph, eager = results
    assert graph.keys() == eager.keys()
    for key in graph:
        assert torch.equal(graph[key], eager[key]), f"graph replay differs from eager launch at {key}"
    everything = dict(requests)
    everything["x"] = extra[: max(p for r, p in graph if r == "x") + 1]
    _compare(graph, everything, weights, cfg, dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_recorded_prompt_steps_match_plain_steps(tmp_path, dtype):
    """Steps whose sizes come again are recorded as graphs and replayed.  The same sequence of
    prompt portions and mixed batches, with other requests, tokens, lengths and pages each time,
    must give the logits of the unrecorded runner, replay after replay, with plain steps and
    synchronisations in between."""
    from mini_llm_runtime_amd.kernels.ops import HipOps

    d = make_model_dir(tmp_path, "A", seed=31)
    cfg, _ = read_weights(d)
    vocab = cfg["vocab_size"]
    outputs = {}
    for use_graphs in (False, True):
        _, _, _, runner = make_runner(d, HipOps(dtype, "cuda"), block_size=BLOCK_SIZE["A"], num_blocks=64, max_requests=4)
        runner.use_graphs = use_graphs
        got = []
        for rnd in range(5):
            a, b = f"a{rnd}", f"b{rnd}"
            runner.cache.create_request(a)
            runner.cache.create_request(b)
            # a prompt step of 40 tokens, a mixed step (a decodes, b brings 23 tokens), a step of two
            # portions of changing split (same totals: same sizes, other lengths), two decode steps
            steps = [
                [StepEntry.of(a, random_tokens(40, vocab, 100 + rnd), (39,))],
                [StepEntry.of(a, random_tokens(1, vocab, 200 + rnd), (0,)), StepEntry.of(b, random_tokens(23, vocab, 300 + rnd), (22,))],
                [StepEntry.of(a, random_tokens(5 + rnd, vocab, 400 + rnd), (0, 4)), StepEntry.of(b, random_tokens(12 - rnd, vocab, 500 + rnd), (3,))],
                [StepEntry.of(a, random_tokens(1, vocab, 600 + rnd), (0,)), StepEntry.of(b, random_tokens(1, vocab, 700 + rnd), (0,))],
            ]
            for entries in steps:
                out = runner.step(entries)
                got.append(out.logits.float().cpu())
                torch.cuda.synchronize()
            runner.cache.release_request(a)
            runner.cache.release_request(b)
        outputs[use_graphs] = got
        if use_graphs:
            assert len(runner._step_graphs) >= 3, "the repeated prompt and mixed steps were not recorded"
        else:
            assert not runner._step_graphs
    for i, (want, have) in enumerate(zip(outputs[False], outputs[True])):
        assert torch.equal(want, have), f"step {i}: a replayed step differs from the plain one"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_half_billion_layer_sizes_match_plain(tmp_path, dtype):
    """Two layers of the Qwen2.5-0.5B sizes (width 896, 14 query and 2 key/value heads of 64,
    feed-forward 4864, vocabulary 151936): the kernels that the large tiles, the long rows of the
    head and prompts of several query tiles select, against the plain implementation; one long
    prompt whole and cut before its last 32 tokens, three shorter ones mixed."""
    from mini_llm_runtime_amd.config.presets import load_preset
    from mini_llm_runtime_amd.kernels.ops import HipOps
    from mini_llm_runtime_amd.models.registry import config_from_dict
    from mini_llm_runtime_amd.weights import write_random_model

    data = load_preset("qwen2.5-0.5b")
    data["num_hidden_layers"] = 2
    config = config_from_dict(data)
    model_dir = write_random_model(config, tmp_path / "half", seed=21, storage_dtype="bfloat16")
    cfg, weights = read_weights(model_dir)
    vocab = cfg["vocab_size"]
    long = {"w": random_tokens(1100, vocab, 700)}
    short = {f"s{i}": random_tokens(n, vocab, 710 + i) for i, n in enumerate((150, 70, 97))}
    _, _, cache, runner = make_runner(model_dir, HipOps(dtype, "cuda"), block_size=16, num_blocks=96, max_requests=4)
    cache.poison()
    for requests, steps in (
        (long, schedules.whole(long)),
        (long, schedules.bulk_then_tail(long)),
        (short, schedules.bulk_then_tail(short)),
        (short, schedules.portions(short)),
        (short, schedules.mixed(short, seed=3)),
    ):
        got = schedules.run_schedule(runner, cache, steps)
        _compare(got, requests, weights, cfg, dtype)
    cache.check_invariants()
    assert cache.request_ids == ()


def _one_layer_of(tmp_path, preset, dtype, seed, lengths):
    """One layer of a large configuration's sizes with a small vocabulary (which keeps the plain
    implementation quick): a long prompt whole, shorter ones in portions down to two tokens, with
    their last tokens one by one, and mixed."""
    from mini_llm_runtime_amd.config.presets import load_preset
    from mini_llm_runtime_amd.kernels.ops import HipOps
    from mini_llm_runtime_amd.models.registry import config_from_dict
    from mini_llm_runtime_amd.weights import write_random_model

    data = load_preset(preset)
    data["num_hidden_layers"] = 1
    data["vocab_size"] = 4099
    config = config_from_dict(data)
    model_dir = write_random_model(config, tmp_path / "large", seed=seed, storage_dtype="bfloat16")
    cfg, weights = read_weights(model_dir)
    long = {"w": random_tokens(lengths[0], cfg["vocab_size"], 720)}
    short = {f"s{i}": random_tokens(n, cfg["vocab_size"], 730 + i) for i, n in enumerate(lengths[1:])}
    _, _, cache, runner = make_runner(model_dir, HipOps(dtype, "cuda"), block_size=16, num_blocks=64, max_requests=4)
    cache.poison()
    for requests, steps in (
        (long, schedules.whole(long)),
        (short, schedules.portions(short)),
        (short, schedules.bulk_then_tail(short, tail=12)),
        (short, schedules.mixed(short, seed=4)),
    ):
        got = schedules.run_schedule(runner, cache, steps)
        _compare(got, requests, weights, cfg, dtype)
    cache.check_invariants()
    assert cache.request_ids == ()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_seven_billion_layer_sizes_match_plain(tmp_path, dtype):
    """Qwen2.5-7B sizes (width 3584, 28 query and 4 key/value heads of 128, feed-forward 18944):
    the largest tiles and the 128-wide heads inside the model."""
    lengths = (700, 90, 40) if dtype == torch.bfloat16 else (300, 70, 40)
    _one_layer_of(tmp_path, "qwen2.5-7b", dtype, 22, lengths)


@pytest.mark.gpu
def test_thirty_two_billion_layer_sizes_match_plain(tmp_path):
    """Qwen2.5-32B sizes (width 5120, 40 query and 8 key/value heads of 128: groups of five;
    feed-forward 27648), bfloat16: 256 x 256 tiles over 55,296 and 27,648 features, a K of 27,648
    cut into slices, decode attention with a group that does not fill its tile."""
    _one_layer_of(tmp_path, "qwen2.5-32b", torch.bfloat16, 23, (600, 90, 40))
