"""The command line: option names and meanings (the reference's where it has them), the
random-model writer, and, on the GPU, generation end to end as child processes."""

from __future__ import annotations

import json
import subprocess
import sys
from pathlib import Path

import pytest

import plain_qwen2 as plain
from helpers import read_weights
from mini_llm_runtime_amd import cli
from mini_llm_runtime_amd.config.presets import load_preset, preset_names

ROOT = Path(__file__).resolve().parents[1]


def test_option_names_follow_the_reference():
    p = cli.build_parser()
    g = p.parse_args(["generate", "--model", "m", "--prompt-ids", "1,2 3", "--max-new-tokens", "4"])
    assert g.prompt_ids == [1, 2, 3] and g.max_new_tokens == 4 and g.temperature == 0.0
    with pytest.raises(SystemExit):  # nothing is ever downloaded: no option that would switch that off
        p.parse_args(["generate", "--model", "m", "--prompt-ids", "1", "--local-files-only"])
    assert p.parse_args(["generate", "--model", "m", "--prompt", "hi"]).max_new_tokens == 8  # the reference's default
    e = p.parse_args(["engine", "--model", "m", "--block-size", "4", "--output-dir", "out"])
    assert e.block_size == 4 and e.output_dir == Path("out") and e.batching_policy == "continuous"
    assert e.dtype is None and e.num_blocks is None and e.kv_memory_fraction == 0.8  # the model folder and free memory decide
    with pytest.raises(SystemExit):  # the reference's choice between its PyTorch paths has nothing to choose here
        p.parse_args(["engine", "--model", "m", "--prefill-attention-backend", "segmented_sdpa"])
    with pytest.raises(SystemExit):
        p.parse_args(["generate", "--prompt-ids", "1"])  # --model is required


def test_presets_and_random_model(tmp_path):
    assert {"qwen2.5-0.5b", "qwen2.5-7b", "qwen2.5-32b", "tiny-a", "tiny-b"} <= set(preset_names())
    half = load_preset("qwen2.5-0.5b")
    assert (half["num_hidden_layers"], half["hidden_size"], half["vocab_size"], half["tie_word_embeddings"]) == (24, 896, 151936, True)
    assert cli.main(["random-model", "--config", "tiny-a", "--seed", "4", "--out", str(tmp_path / "m")]) == 0
    cfg, w = read_weights(tmp_path / "m")
    assert cfg["architectures"] == ["Qwen2ForCausalLM"] and w["model.embed_tokens.weight"].shape == (256, 64)
    with pytest.raises(FileNotFoundError, match="presets"):
        load_preset("no-such-model")


@pytest.mark.gpu
def test_generate_and_engine_commands(tmp_path, gpu_device):
    model = tmp_path / "m"
    run = lambda *a: subprocess.run([sys.executable, "-m", "mini_llm_runtime_amd.cli", *a], cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert run("random-model", "--config", "tiny-b", "--seed", "9", "--out", str(model)).returncode == 0
    cfg, w = read_weights(model)
    prompt = [5, 17, 3, 200, 41, 77, 9]
    proc = run("generate", "--model", str(model), "--dtype", "float32", "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "6")
    assert proc.returncode == 0, proc.stderr[-2000:]
    out = json.loads(proc.stdout.strip().splitlines()[-1])
    assert out["generated_token_ids"] == plain.greedy(prompt, w, cfg, 6)
    assert out["prefill_tokens"] == 7 and out["decode_steps"] == 5 and out["cache_length"] == 12
    sampled = run("generate", "--model", str(model), "--dtype", "float32", "--prompt-ids", "5,17,3", "--max-new-tokens", "8",
                  "--temperature", "0.9", "--seed", "3")
    again = run("generate", "--model", str(model), "--dtype", "float32", "--prompt-ids", "5,17,3", "--max-new-tokens", "8",
                "--temperature", "0.9", "--seed", "3")
    assert sampled.returncode == 0 and sampled.stdout == again.stdout
    proc = run("engine", "--model", str(model), "--block-size", "4", "--num-blocks", "16", "--output-dir", str(tmp_path / "out"))
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "all KV blocks released = True" in proc.stdout
    result = json.loads((tmp_path / "out" / "result.json").read_text())
    assert result["all_resources_released"] and (tmp_path / "out" / "report.md").is_file()
    for r in result["requests"]:
        assert result["generated_token_ids"][r["id"]] == plain.greedy(r["prompt_ids"], w, cfg, r["max_new_tokens"])
    assert any(s["prefill"] and s["decode"] for s in result["steps"]), "the demonstration should hold a mixed step"
    missing = run("generate", "--model", str(tmp_path / "nothing"), "--prompt-ids", "1")
    assert missing.returncode != 0 and "config.json" in missing.stderr
