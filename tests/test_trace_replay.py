"""Trace replay: the same requests whole, with the last 32 tokens one by one, in
portions of changing size, and mixed so that pages are used again, all compared with
the plain implementation.  The replay loop runs on the CPU with the torch stand-in;
`bin/trace_run` itself runs on the GPU as a child process, in 32-bit and bfloat16."""

from __future__ import annotations

import io
import json
import subprocess
from pathlib import Path

import numpy as np
import pytest
import torch

import mini_llm_runtime_amd as mlr
import plain_qwen2 as plain
import schedules
from helpers import TINY, make_model_dir, random_tokens, read_weights
from kernel_doubles import TorchOps
from mini_llm_runtime_amd.engine import ModelRunner
from mini_llm_runtime_amd.replay import PAGE_TOKENS, TraceError, replay

ROOT = Path(__file__).resolve().parents[1]
LENGTHS = {"A": (40, 75, 33, 130, 64, 90), "B": (36, 63, 100, 41, 77, 50), "C": (35, 70, 99, 44, 65, 38), "D": (37, 66, 34, 101, 52, 40)}


def _requests(which):
    vocab = TINY[which]["vocab_size"]
    return {f"q{i}": random_tokens(n, vocab, 300 + i) for i, n in enumerate(LENGTHS[which])}


def _max_tokens(steps, rounding=64):
    """Most tokens live requests hold at any time, each request's count rounded up to 64."""
    fed, most = {}, 0
    for step in steps:
        for e in step["entries"]:
            fed[e["id"]] = fed.get(e["id"], 0) + len(e["tokens"])
        most = max(most, sum(-(-n // rounding) * rounding for n in fed.values()))
        for rid in step["end"]:
            fed.pop(rid, None)
    return most


def _collect(steps, out_dir, vocab):
    got, fed = {}, {}
    for step in steps:
        wanted = [(e["id"], fed.get(e["id"], 0) + w) for e in step["entries"] for w in e["want"]]
        path = Path(out_dir) / f"{step['step']}.f32"
        if wanted:
            rows = np.fromfile(path, dtype="<f4").reshape(len(wanted), vocab)
            for key, row in zip(wanted, rows):
                got[key] = torch.from_numpy(row.copy())
        else:
            assert not path.exists()
        for e in step["entries"]:
            fed[e["id"]] = fed.get(e["id"], 0) + len(e["tokens"])
        for rid in step["end"]:
            fed.pop(rid, None)
    return got


def _compare(got, requests, weights, cfg, dtype):
    num = den = worst = worst_row = 0.0
    for rid, toks in requests.items():
        ref = plain.forward(toks, weights, cfg)
        for pos in range(len(toks)):
            diff = got[(rid, pos)].double() - ref[pos]
            worst = max(worst, float(diff.abs().max()))
            worst_row = max(worst_row, float(diff.norm() / ref[pos].norm()))
            num += float((diff**2).sum())
            den += float((ref[pos] ** 2).sum())
    if dtype == "float32":
        assert worst < 1e-4, worst
    else:
        assert (num / den) ** 0.5 < 2e-2, (num / den) ** 0.5
        assert worst_row < 5e-2, worst_row  # no single position may hide in the aggregate


FAMILIES = {
    "whole": schedules.whole,
    "bulk_then_tail": schedules.bulk_then_tail,
    "portions": schedules.portions,
    "mixed": lambda r: schedules.mixed(r, seed=9),
}


@pytest.mark.parametrize("family", list(FAMILIES))
def test_replay_loop_on_cpu(tmp_path, family):
    d = make_model_dir(tmp_path, "B", seed=31)
    cfg, w = read_weights(d)
    requests = _requests("B")
    steps = FAMILIES[family](requests)
    ops = TorchOps(torch.float32)
    _, model = mlr.load_model(d, dtype=torch.float32, device="cpu")
    cache = mlr.make_cache(model, block_size=PAGE_TOKENS, num_blocks=-(-_max_tokens(steps) // PAGE_TOKENS), max_requests=8)
    cache.poison()
    done = io.StringIO()
    lines = io.StringIO("\n".join(json.dumps(s) for s in steps) + "\n")
    assert replay(ModelRunner(model, cache, ops), cache, lines, tmp_path / "out", done) == len(steps)
    assert done.getvalue().split("\n")[:-1] == [f"done {s['step']}" for s in steps]
    _compare(_collect(steps, tmp_path / "out", cfg["vocab_size"]), requests, w, cfg, "float32")
    assert cache.request_ids == ()


def test_replay_rejects_bad_lines(tmp_path):
    d = make_model_dir(tmp_path, "A", seed=32)
    _, model = mlr.load_model(d, dtype=torch.float32, device="cpu")
    cache = mlr.make_cache(model, block_size=PAGE_TOKENS, num_blocks=4, max_requests=8)
    runner = ModelRunner(model, cache, TorchOps(torch.float32))
    for line in ("not json", '{"entries": []}', '{"step": 0, "entries": [{"id": "a", "tokens": []}]}'):
        with pytest.raises(TraceError):
            replay(runner, cache, io.StringIO(line + "\n"), tmp_path / "o", io.StringIO())
    with pytest.raises(ValueError, match="vocabulary"):
        replay(runner, cache, io.StringIO('{"step": 0, "entries": [{"id": "a", "tokens": [99999]}]}\n'), tmp_path / "o", io.StringIO())
    assert cache.request_ids == ()  # the failed step left nothing behind


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C", "D"])
def test_trace_run_program(tmp_path, gpu_device, which, dtype):
    d = make_model_dir(tmp_path, which, seed=33)
    cfg, w = read_weights(d)
    requests = _requests(which)
    for family, make in FAMILIES.items():
        steps = make(requests)
        out = tmp_path / f"out_{family}"
        proc = subprocess.run(
            [str(ROOT / "bin" / "trace_run"), "--model", str(d), "--dtype", dtype, "--out", str(out),
             "--max-tokens", str(_max_tokens(steps))],
            input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300,
        )
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert proc.stdout.split() == [x for s in steps for x in ("done", str(s["step"]))]
        _compare(_collect(steps, out, cfg["vocab_size"]), requests, w, cfg, dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("block_size", [8, 32, 128])
def test_trace_run_program_at_other_page_sizes(tmp_path, gpu_device, block_size, dtype):
    """The program itself (not only the step function) with pages of 8, 32 and 128 tokens; a
    page larger than 64 tokens is what the caller rounds every request up to."""
    d = make_model_dir(tmp_path, "B", seed=34)
    cfg, w = read_weights(d)
    requests = _requests("B")
    for family in ("portions", "mixed"):
        steps = FAMILIES[family](requests)
        out = tmp_path / f"out_{family}"
        proc = subprocess.run(
            [str(ROOT / "bin" / "trace_run"), "--model", str(d), "--dtype", dtype, "--out", str(out),
             "--max-tokens", str(_max_tokens(steps, max(64, block_size))), "--block-size", str(block_size)],
            input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300,
        )
        assert proc.returncode == 0, proc.stderr[-2000:]
        _compare(_collect(steps, out, cfg["vocab_size"]), requests, w, cfg, dtype)


def _site_reference(toks, w, cfg):
    x = w["model.embed_tokens.weight"].double()[torch.tensor(toks)]
    wd = {k: v.double() for k, v in w.items()}
    out = []
    for i in range(cfg["num_hidden_layers"]):
        x = plain.decoder_layer(x, torch.arange(len(toks)), wd, i, cfg)
        out.append(x)
    return torch.stack(out)


def test_replay_writes_the_stream_after_every_site(tmp_path):
    """`--layers`: <step>.layers.f32 holds [sites, wanted, hidden], the plain layers' outputs."""
    d = make_model_dir(tmp_path, "A", seed=35)
    cfg, w = read_weights(d)
    toks = random_tokens(21, cfg["vocab_size"], 36)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": toks[:13], "want": [0, 12]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": toks[13:20], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": toks[20:], "want": [0]}], "end": ["a"]},
    ]
    _, model = mlr.load_model(d, dtype=torch.float32, device="cpu")
    cache = mlr.make_cache(model, block_size=PAGE_TOKENS, num_blocks=2, max_requests=1)
    lines = io.StringIO("\n".join(json.dumps(s) for s in steps) + "\n")
    replay(ModelRunner(model, cache, TorchOps(torch.float32)), cache, lines, tmp_path / "o", io.StringIO(), layers=True)
    ref = _site_reference(toks, w, cfg)
    layers, hidden = cfg["num_hidden_layers"], cfg["hidden_size"]
    first = torch.from_numpy(np.fromfile(tmp_path / "o" / "0.layers.f32", dtype="<f4").reshape(layers, 2, hidden).copy())
    assert float((first.double() - ref[:, [0, 12]]).abs().max()) < 1e-5
    assert not (tmp_path / "o" / "1.layers.f32").exists() and not (tmp_path / "o" / "1.f32").exists()
    last = torch.from_numpy(np.fromfile(tmp_path / "o" / "2.layers.f32", dtype="<f4").reshape(layers, 1, hidden).copy())
    assert float((last.double() - ref[:, [20]]).abs().max()) < 1e-5


def test_replay_names_the_limit_on_live_requests(tmp_path):
    d = make_model_dir(tmp_path, "A", seed=37)
    _, model = mlr.load_model(d, dtype=torch.float32, device="cpu")
    cache = mlr.make_cache(model, block_size=PAGE_TOKENS, num_blocks=8, max_requests=2)
    runner = ModelRunner(model, cache, TorchOps(torch.float32))
    steps = [{"step": i, "entries": [{"id": f"r{i}", "tokens": [1, 2], "want": []}], "end": []} for i in range(3)]
    with pytest.raises(TraceError, match="--max-live is 2"):
        replay(runner, cache, io.StringIO("\n".join(json.dumps(s) for s in steps) + "\n"), tmp_path / "o", io.StringIO())
    assert set(cache.request_ids) == {"r0", "r1"}  # the steps before the refused one stand


@pytest.mark.gpu
def test_trace_run_program_writes_layers(tmp_path, gpu_device):
    d = make_model_dir(tmp_path, "B", seed=38)
    cfg, w = read_weights(d)
    toks = random_tokens(40, cfg["vocab_size"], 39)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": toks[:33], "want": [32]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": toks[33:], "want": [0, 6]}], "end": ["a"]},
    ]
    proc = subprocess.run(
        [str(ROOT / "bin" / "trace_run"), "--model", str(d), "--dtype", "float32", "--out", str(tmp_path / "o"),
         "--max-tokens", "64", "--layers"],
        input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300,
    )
    assert proc.returncode == 0, proc.stderr[-2000:]
    ref = _site_reference(toks, w, cfg)
    got = np.fromfile(tmp_path / "o" / "1.layers.f32", dtype="<f4").reshape(cfg["num_hidden_layers"], 2, cfg["hidden_size"])
    assert float((torch.from_numpy(got.copy()).double() - ref[:, [33, 39]]).abs().max()) < 1e-4
