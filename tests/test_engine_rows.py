"""Rows of the engine that have no test file of their own: the engine's configuration, the
residual stream captured after every site, the debug check on reads of pending tokens, the
lifetime of a step's logits, and the own safetensors reader and writer against the
`safetensors` library."""

from __future__ import annotations

import json

import pytest
import torch

import mini_llm_runtime_amd as mlr
import plain_qwen2 as plain
from helpers import BLOCK_SIZE, StepEntry, make_model_dir, make_runner, random_tokens, read_weights
from kernel_doubles import TorchOps
from mini_llm_runtime_amd.cache import PagedKVSpec, VisibilityError
from mini_llm_runtime_amd.engine import ContinuousBatchEngine, EngineConfig, GraphLimits, ModelRunner
from mini_llm_runtime_amd.engine.config import blocks_for_memory, dtype_of_checkpoint
from mini_llm_runtime_amd.engine.factory import page_bytes
from mini_llm_runtime_amd.kernels.tuning import KernelTuning
from mini_llm_runtime_amd.parts.context import KVView
from mini_llm_runtime_amd.weights.safetensors_io import SafetensorsFile, write_safetensors

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


# ---- configuration of the engine -----------------------------------------------------------------------
def test_engine_config_defaults_overrides_and_checks():
    c = EngineConfig()
    assert (c.block_size, c.max_running_requests, c.max_batch_tokens, c.num_blocks) == (16, 8, 2048, None)
    assert c.dtype is None and c.graphs == GraphLimits() and c.tuning == KernelTuning()
    assert c.resolved_dtype({"torch_dtype": "float32"}) is torch.float32
    assert c.resolved_dtype({"torch_dtype": "bfloat16"}) is torch.bfloat16
    assert c.resolved_dtype({"torch_dtype": "float16"}) is torch.bfloat16  # no float16 path
    assert dtype_of_checkpoint({}) is torch.bfloat16
    assert c.with_overrides(dtype="float32").resolved_dtype({"torch_dtype": "bfloat16"}) is torch.float32
    d = c.with_overrides(block_size=4, num_blocks=9)
    assert (d.block_size, d.num_blocks) == (4, 9) and c.block_size == 16
    with pytest.raises(TypeError, match="no_such"):
        c.with_overrides(no_such=1)
    for bad in (dict(block_size=0), dict(num_blocks=0), dict(kv_memory_fraction=0.0), dict(kv_memory_fraction=1.5),
                dict(dtype="float16"), dict(batching_policy="continuous"), dict(max_batch_tokens=True)):
        with pytest.raises(ValueError):
            EngineConfig(**bad)
    with pytest.raises(ValueError):
        GraphLimits(max_decode_graphs=0)
    with pytest.raises(ValueError):
        KernelTuning(decode_partition=0)
    assert blocks_for_memory(1000, 10_000, 0.55) == 5
    with pytest.raises(ValueError, match="hold no page"):
        blocks_for_memory(1000, 900, 1.0)


def test_engine_from_model_dir_takes_the_config(tmp_path):
    d = make_model_dir(tmp_path, "A", seed=61, storage_dtype="float32")
    assert json.loads((d / "config.json").read_text())["torch_dtype"] == "float32"
    ops = TorchOps(torch.float32, "cpu")
    config = EngineConfig(block_size=4, num_blocks=12, max_running_requests=3, max_batch_tokens=16,
                          graphs=GraphLimits(enabled=False, max_decode_batch=32))
    engine = ContinuousBatchEngine.from_model_dir(d, config, ops=ops, max_batch_tokens=24)
    assert engine.config.max_batch_tokens == 24 and engine.config.block_size == 4
    assert engine.manager.block_size == 4 and engine.manager.groups[0].num_blocks == 12
    assert engine.scheduler.max_running_requests == 3 and engine.scheduler.max_batch_tokens == 24
    assert engine.runner.max_graph_batch == 32 and not engine.runner.use_graphs
    assert engine.runner.dtype is torch.float32  # from config.json's torch_dtype: nothing else named one
    _, model = mlr.load_model(d, dtype=torch.float32, device="cpu")
    # keys and values of 2 layers x 2 kv heads x head size 16 x 4 tokens x 4 bytes
    assert page_bytes(model, 4, torch.float32) == 2 * 2 * 2 * 16 * 4 * 4
    with pytest.raises(ValueError, match="needs a GPU"):
        ContinuousBatchEngine.from_model_dir(d, EngineConfig(), ops=ops)  # no num_blocks, no GPU to size by


@pytest.mark.gpu
def test_page_pool_from_free_memory_and_dtype_from_the_folder(tmp_path, gpu_device):
    d = make_model_dir(tmp_path, "B", seed=62, storage_dtype="float32")
    free, _ = torch.cuda.mem_get_info()
    engine = ContinuousBatchEngine.from_model_dir(d, EngineConfig(block_size=8, kv_memory_fraction=0.01))
    assert engine.runner.dtype is torch.float32
    _, model = mlr.load_model(d, dtype=torch.float32, device="cuda")
    pages = engine.manager.groups[0].num_blocks
    per_page = page_bytes(model, 8, torch.float32)
    assert 0.005 * free < pages * per_page <= 0.01 * free
    cfg, w = read_weights(d)
    prompt = random_tokens(11, cfg["vocab_size"], 3)
    assert engine.generate([prompt], max_new_tokens=4)[0] == plain.greedy(prompt, w, cfg, 4)


def test_memory_set_aside_for_recorded_steps(tmp_path):
    """The page pool is sized from what is free after the weights less an estimate of what
    recorded steps will hold: nothing without recordings, more with more or larger ones."""
    from mini_llm_runtime_amd.engine.factory import recording_reserve_bytes

    d = make_model_dir(tmp_path, "A", seed=64)
    cfg, _ = read_weights(d)
    _, model = mlr.load_model(d, dtype=torch.float32, device="cpu")
    base = recording_reserve_bytes(model, GraphLimits(), torch.bfloat16, 8, 2048)
    assert recording_reserve_bytes(model, GraphLimits(enabled=False), torch.bfloat16, 8, 2048) == 0
    assert recording_reserve_bytes(model, None, torch.bfloat16, 8, 2048) == 0
    # at least the logits of one recording per padded batch size 1, 2, 4, 8
    assert base >= (1 + 2 + 4 + 8) * cfg["vocab_size"] * 4
    assert recording_reserve_bytes(model, GraphLimits(max_step_graphs=32), torch.bfloat16, 8, 2048) > base
    assert recording_reserve_bytes(model, GraphLimits(), torch.bfloat16, 64, 2048) > base
    assert recording_reserve_bytes(model, GraphLimits(), torch.bfloat16, 8, 8192) > base
    assert recording_reserve_bytes(model, GraphLimits(), torch.float32, 8, 2048) > base


@pytest.mark.gpu
def test_a_recording_that_runs_out_of_memory_falls_back_to_plain_steps(tmp_path, gpu_device, monkeypatch):
    """The condition is forced from the host (the graph object refuses to be made); the step must
    still give the right logits, recordings must be off afterwards, and one warning says so."""
    d = make_model_dir(tmp_path, "A", seed=65)
    cfg, w = read_weights(d)
    _, _, _, runner = make_runner(d, _ops("hip", torch.float32), block_size=BLOCK_SIZE["A"], num_blocks=16)
    tokens = random_tokens(9, cfg["vocab_size"], 4)
    ref = plain.forward(tokens, w, cfg)
    runner.cache.create_request("r")
    runner.step([StepEntry.of("r", tokens[:8], [7])])
    assert runner.use_graphs

    def no_memory(*args, **kwargs):
        raise torch.cuda.OutOfMemoryError("forced by the test")

    monkeypatch.setattr(torch.cuda, "CUDAGraph", no_memory)
    with pytest.warns(RuntimeWarning, match="recordings are switched off"):
        out = runner.step([StepEntry.of("r", tokens[8:], [0])])  # a single token: would be recorded
    assert not runner.use_graphs and not runner._graphs
    torch.testing.assert_close(out.logits[0].double().cpu(), ref[8], atol=1e-4, rtol=1e-4)
    assert runner.cache.get_request("r").num_tokens == 9 and not runner.cache.step_in_flight


# ---- the residual stream after every site -------------------------------------------------------------------
@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("which", ["A", "B"])
def test_site_outputs_match_the_plain_layers(tmp_path, which, backend, dtype):
    """`capture_sites` returns what the reference's `return_layer_outputs` does
    (src/mini_llm_runtime/qwen_model_runner.py:266-281): the stream after each layer.  A prompt
    in two portions and then single tokens, every site compared with the plain layer stack."""
    d = make_model_dir(tmp_path, which, seed=63)
    cfg, w = read_weights(d)
    ops = _ops(backend, dtype)
    _, _, cache, runner = make_runner(d, ops, block_size=BLOCK_SIZE[which], num_blocks=16)
    cache.poison()
    toks = random_tokens(30, cfg["vocab_size"], 64)
    x = w["model.embed_tokens.weight"].double()[torch.tensor(toks)]
    positions = torch.arange(len(toks))
    expected = []
    wd = {k: v.double() for k, v in w.items()}
    for i in range(cfg["num_hidden_layers"]):
        x = plain.decoder_layer(x, positions, wd, i, cfg)
        expected.append(x)
    expected = torch.stack(expected)  # [layers, tokens, hidden]
    cache.create_request("r")
    at = 0
    for n, want in ((17, (0, 5, 16)), (9, (0, 8)), (1, (0,)), (1, (0,)), (1, (0,))):
        out = runner.step([StepEntry.of("r", toks[at : at + n], want)], capture_sites=True)
        assert out.site_outputs.shape == (cfg["num_hidden_layers"], len(want), cfg["hidden_size"])
        assert out.site_outputs.dtype == torch.float32
        ref = expected[:, [at + i for i in want]]
        err = (out.site_outputs.double().cpu() - ref).abs().max() / ref.abs().max()
        assert float(err) < (1e-5 if dtype == torch.float32 else 3e-2), (at, float(err))
        plain_logits = plain.forward(toks[: at + n], w, cfg)[[at + i for i in want]]
        bound = 1e-4 if dtype == torch.float32 else 0.05 * float(plain_logits.abs().max())
        assert float((out.logits.double().cpu() - plain_logits).abs().max()) < bound
        at += n
    nothing = runner.step([StepEntry.of("r", toks[at : at + 1], ())], capture_sites=True)
    assert nothing.site_outputs is None and nothing.logits is None
    cache.release_request("r")


# ---- reads of pending tokens before their write ------------------------------------------------------------------
def test_visibility_check_on_the_manager():
    spec = PagedKVSpec(1, 8)
    m = mlr.CacheManager([spec, None, spec], block_size=4, num_blocks=4, max_requests=2, dtype=torch.float32,
                         device="cpu", check_visibility=True)
    view = lambda site, owner: KVView(None, None, None, None, 4, None, site == owner, site=site, owner=owner,
                                      tracker=m.visibility_tracker)
    with pytest.raises(VisibilityError, match="outside a step"):
        view(0, 0).written()
    m.create_request("a")
    m.begin_step([("a", 3)])
    with pytest.raises(VisibilityError, match="before they were written"):
        view(0, 0).reading()
    view(0, 0).written()
    view(0, 0).reading()
    view(1, 0).reading()  # a site that reads site 0's pages: fine once site 0 has written
    with pytest.raises(VisibilityError, match="only reads"):
        view(1, 0).written()
    with pytest.raises(VisibilityError, match=r"sites \[2\]"):
        m.commit_step()  # site 2 owns pages and never wrote
    assert m.step_in_flight and m.get_request("a").num_tokens == 0  # the refused commit changed nothing
    view(2, 2).written()
    m.commit_step()
    assert m.get_request("a").num_tokens == 3
    m.begin_step([("a", 1)])  # a new step starts with nothing written
    with pytest.raises(VisibilityError):
        view(2, 2).reading()
    m.abort_step()
    quiet = mlr.CacheManager([spec], block_size=4, num_blocks=4, max_requests=2, dtype=torch.float32, device="cpu")
    assert quiet.visibility_tracker is None  # without the flag a view reports to nobody


def test_a_mixer_that_skips_its_write_is_caught(tmp_path):
    """The model's own attention part reports its write and its read; one that forgets the
    write (here: the report is dropped) cannot read the step's tokens and cannot commit."""
    from mini_llm_runtime_amd.engine.factory import load_model, make_cache

    d = make_model_dir(tmp_path, "A", seed=65)
    cfg, w = read_weights(d)
    ops = TorchOps(torch.float32, "cpu")
    _, model = load_model(d, dtype=torch.float32, device="cpu")
    cache = make_cache(model, block_size=4, num_blocks=8, max_requests=2, check_visibility=True)
    runner = ModelRunner(model, cache, ops)
    toks = random_tokens(6, cfg["vocab_size"], 66)
    cache.create_request("ok")
    out = runner.step([StepEntry.of("ok", toks, (5,))])  # the real parts pass the check
    assert float((out.logits[0].double() - plain.forward(toks, w, cfg)[-1]).abs().max()) < 1e-4
    original = KVView.written
    KVView.written = lambda self: None  # the part "forgets" to write
    try:
        cache.create_request("bad")
        with pytest.raises(VisibilityError, match="before they were written"):
            runner.step([StepEntry.of("bad", toks, (5,))])
    finally:
        KVView.written = original
    assert not cache.step_in_flight and cache.get_request("bad").num_tokens == 0
    cache.check_invariants()


# ---- how long a step's logits live -------------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_logits_of_a_step_survive_the_next_steps(tmp_path, gpu_device, dtype):
    """Steps that replay a recording hand out copies; `borrow_logits=True` hands out the
    recording's own buffer, which the next replay overwrites."""
    from mini_llm_runtime_amd.kernels.ops import HipOps

    d = make_model_dir(tmp_path, "B", seed=67)
    cfg, _ = read_weights(d)
    _, _, cache, runner = make_runner(d, HipOps(dtype, "cuda"), block_size=8, num_blocks=32)
    toks = random_tokens(40, cfg["vocab_size"], 68)
    cache.create_request("r")
    runner.step([StepEntry.of("r", toks[:20], ())])
    kept, copies = [], []
    for t in toks[20:30]:  # single-token steps: recorded at the first, replayed from then on
        out = runner.step([StepEntry.of("r", [t], (0,))])
        kept.append(out.logits)
        copies.append(out.logits.clone())
    assert runner._graphs, "the decode steps were not recorded"
    for i, (a, b) in enumerate(zip(kept, copies)):
        assert torch.equal(a, b), f"the logits of step {i} changed after later steps"
    assert len({t.data_ptr() for t in kept}) == len(kept)
    first = runner.step([StepEntry.of("r", [toks[30]], (0,))], borrow_logits=True).logits
    before = first.clone()
    second = runner.step([StepEntry.of("r", [toks[31]], (0,))], borrow_logits=True).logits
    assert first.data_ptr() == second.data_ptr() and not torch.equal(first, before)  # documented: borrowed = overwritten
    cache.release_request("r")


# ---- the own safetensors code against the library ---------------------------------------------------------------------------
def test_safetensors_files_agree_with_the_safetensors_library(tmp_path):
    """Both directions: what `write_safetensors` wrote the library reads back bit for bit, and
    what the library wrote `SafetensorsFile` reads back bit for bit (bfloat16, float32, int32,
    int64, a scalar-like and an empty-ish shape, metadata)."""
    st = pytest.importorskip("safetensors.torch")
    from safetensors import safe_open

    g = torch.Generator().manual_seed(5)
    tensors = {
        "a.weight": torch.randn(7, 5, generator=g).to(torch.bfloat16),
        "b.bias": torch.randn(13, generator=g),
        "c.table": torch.randint(-1000, 1000, (3, 4), generator=g, dtype=torch.int32),
        "d.long": torch.randint(-(2**40), 2**40, (6,), generator=g, dtype=torch.int64),
        "e.one": torch.randn(1, generator=g),
        "f.wide": torch.randn(2, 3, 4, generator=g).to(torch.bfloat16),
    }
    ours = tmp_path / "ours.safetensors"
    write_safetensors(ours, [(n, t.dtype, tuple(t.shape)) for n, t in tensors.items()], iter(tensors.items()),
                      metadata={"format": "pt", "note": "x"})
    with safe_open(str(ours), framework="pt") as f:
        assert set(f.keys()) == set(tensors) and f.metadata() == {"format": "pt", "note": "x"}
        for name, t in tensors.items():
            back = f.get_tensor(name)
            assert back.dtype == t.dtype and back.shape == t.shape and torch.equal(back, t), name
    theirs = tmp_path / "theirs.safetensors"
    st.save_file(tensors, str(theirs), metadata={"format": "pt"})
    with SafetensorsFile(theirs) as f:
        assert set(f.entries) == set(tensors)
        for name, t in tensors.items():
            back = f.tensor(name)
            want = t.to(torch.int32) if t.dtype == torch.int64 and back.dtype == torch.int32 else t
            assert back.shape == t.shape and torch.equal(back.to(want.dtype), want), name


# ---- the attention kernels' plan ------------------------------------------------------------------------
def test_attention_plan_covers_every_query_once_in_both_tile_sizes():
    """Both tile lists of the plan (64 and 128 queries) cover every token of every entry with more
    than one new token exactly once, heaviest tiles first; single-token entries are only counted."""
    import numpy as np

    from mini_llm_runtime_amd.kernels.plans import QUERY_TILE, WIDE_QUERY_TILE, attention_plan
    from mini_llm_runtime_amd.parts.context import PlanInput

    q_lens = np.array([1, 300, 64, 1, 129, 2], dtype=np.int32)
    q_starts = np.array([77, 0, 500, 9, 130, 4000], dtype=np.int32)
    plan = attention_plan(PlanInput(q_lens, q_starts, 4096))
    assert plan.sizes["num_decode_entries"] == 2 and plan.sizes["max_decode_context"] == 4096
    for name, count, tile in (("query_tiles", "num_query_tiles", QUERY_TILE), ("wide_query_tiles", "num_wide_query_tiles", WIDE_QUERY_TILE)):
        tiles = plan.arrays[name]
        assert plan.sizes[count] == len(tiles)
        covered = {r: np.zeros(n, dtype=int) for r, n in enumerate(q_lens) if n > 1}
        for entry, q0 in tiles:
            covered[int(entry)][q0 : q0 + tile] += 1
        assert all((c == 1).all() for c in covered.values()), name
        weights = [int(q_starts[e]) + int(q0) for e, q0 in tiles]
        assert weights == sorted(weights, reverse=True), "tiles with the most keys before them come first"
    assert plan.sizes["long_prefix"] == 0
    behind = attention_plan(PlanInput(np.array([512, 1], dtype=np.int32), np.array([6000, 9000], dtype=np.int32), 16384))
    assert behind.sizes["long_prefix"] == 2, "a portion behind 6,000 cached tokens"
    nearer = attention_plan(PlanInput(np.array([512], dtype=np.int32), np.array([3000], dtype=np.int32), 16384))
    assert nearer.sizes["long_prefix"] == 1, "a portion behind 3,000 cached tokens"
    no_prompts = attention_plan(PlanInput(np.ones(3, dtype=np.int32), np.zeros(3, dtype=np.int32), 64))
    assert no_prompts.sizes["num_query_tiles"] == 0 and no_prompts.arrays["wide_query_tiles"].shape == (0, 2)
