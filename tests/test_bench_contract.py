"""The measurement program's contract: one GPU only, and a line that names every size."""

from __future__ import annotations

import json
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]


def test_more_than_one_gpu_is_refused_with_one_line():
    run = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert run.returncode == 2
    lines = [l for l in (run.stdout + run.stderr).splitlines() if l.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


@pytest.mark.gpu
def test_default_line_keeps_the_contract(tmp_path):
    """A short run at the default shape (fewer steps, no larger shapes): the line has the metric,
    the timing fields, a flat configuration of at most 20 keys that names every size, the prefill
    and the roofline of the decode step."""
    run = subprocess.run(
        [sys.executable, str(ROOT / "bench.py"), "--steps", "8", "--warmup", "2", "--no-large"],
        capture_output=True, text=True, timeout=600, cwd=str(ROOT),
    )
    assert run.returncode == 0, run.stderr[-2000:]
    lines = [l for l in run.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    line = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 8 and line["warmup"] == 2 and line["higher_is_better"] is True
    assert abs(line["value"] - 8e3 / line["ms_per_step"]) < 0.01 * line["value"]
    config = line["config"]
    assert len(config) <= 20 and all(not isinstance(v, (dict, list)) for v in config.values())
    for size in ("hidden_size", "num_attention_heads", "num_key_value_heads", "head_dim", "intermediate_size",
                 "vocab_size", "layers", "layers_full_model", "global_batch", "seq_len"):
        assert size in config, size
    assert config["layers"] == config["layers_full_model"] == 24 and config["global_batch"] == 8
    assert line["prefill"]["tokens"] == 2048 and 0 < line["prefill"]["frac"] < 1
    roof = line["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert set(line["points"]) == {"decode_b1", "decode_b64"}
    memory = line["peak_memory_gb"]  # weights (about 1 GB) and the page pool at least, the card's 288 GB at most
    assert 1.0 < memory["allocated"] <= memory["reserved"] < 288 and memory["device_in_use"] >= memory["reserved"]


@pytest.mark.gpu
def test_the_reference_measurements_workload_prints_its_line():
    """The reference's published measurements at their parameters: both batching policies of the burst of
    eight, the 4 x 512 prompt step and the decode attention, each beside the published figure."""
    run = subprocess.run(
        [sys.executable, str(ROOT / "bench.py"), "--workload", "reference"],
        capture_output=True, text=True, timeout=600, cwd=str(ROOT),
    )
    assert run.returncode == 0, run.stderr[-2000:]
    lines = [l for l in run.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    line = json.loads(lines[0])
    bursts = line["burst_of_8"]
    assert set(bursts) == {"continuous", "static"}
    for policy in bursts.values():
        assert policy["tokens_per_s"] > 0 and policy["median_ttft_ms"] > 0 and policy["median_e2e_ms"] >= policy["median_ttft_ms"]
    # a request of the second batch waits for the whole first batch under static batching
    assert bursts["static"]["median_ttft_ms"] > bursts["continuous"]["median_ttft_ms"]
    assert line["value"] == bursts["continuous"]["tokens_per_s"]
    assert abs(line["vs_baseline"] - line["value"] / line["published"]["continuous"]["tokens_per_s"]) < 0.1
    assert line["prefill_4x512_ms"] > 0 and line["decode_attention_us"] > 0
    # with every page reserved the late request waits for a request to finish: one step longer in the queue
    late = line["late_request_under_page_pressure"]
    assert late["28_blocks"]["queue_wait_ms"] > late["29_blocks"]["queue_wait_ms"] and late["paired_ttft_difference_ms"] > 0
