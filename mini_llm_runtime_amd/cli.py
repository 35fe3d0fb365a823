"""Command line.

    python -m mini_llm_runtime_amd.cli generate --model DIR --prompt-ids 1,2,3 --max-new-tokens 8
    python -m mini_llm_runtime_amd.cli engine   --model DIR --block-size 16 --output-dir OUT
    python -m mini_llm_runtime_amd.cli random-model --config qwen2.5-0.5b --seed 0 --out DIR

`generate` follows the reference's `experiments/greedy_generation_runner.py:19-25`
(`--model`, `--prompt`, `--max-new-tokens`); `engine` follows its
`experiments/continuous_batch_engine_runner.py:32-52` (`--model`, `--block-size`,
`--output-dir`) and runs the same kind of demonstration: requests that join and leave a
running batch, with a record of every step.  Options of the reference without a
counterpart: `--local-files-only` (its `--model` may name a hub repository to download;
`--model` here is a folder and nothing is ever fetched, so there is nothing to switch off)
and `--prefill-attention-backend` / `--prefill-kv-write-backend` (they choose between its
PyTorch code paths; this engine has one kernel path).
`--dtype` defaults to what the model folder's config.json says (`torch_dtype`); the page
pool is `--num-blocks` pages or, without it, `--kv-memory-fraction` of the free device memory.

Tokens in, tokens out: the engine has no tokenizer of its own (the reference's
scripts borrow an external one).  `--prompt` is accepted when the model folder
holds a `tokenizer.json` and the `tokenizers` package is importable; otherwise
give `--prompt-ids`.
"""

from __future__ import annotations

import argparse
import json
import sys
from dataclasses import asdict
from pathlib import Path
from typing import Any, Optional, Sequence


def _add_model_options(p: argparse.ArgumentParser) -> None:
    p.add_argument("--model", required=True, type=Path, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", default=None, choices=("bfloat16", "float32"), help="default: config.json's torch_dtype")


def _ids(text: str) -> list[int]:
    try:
        return [int(t) for t in text.replace(",", " ").split()]
    except ValueError:
        raise argparse.ArgumentTypeError("token ids are integers separated by commas or spaces") from None


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="mini_llm_runtime_amd", description=__doc__.split("\n\n")[0])
    sub = parser.add_subparsers(dest="command", required=True)

    g = sub.add_parser("generate", help="one request: prompt step, then one token per step")
    _add_model_options(g)
    g.add_argument("--prompt", help="text prompt (needs tokenizer.json in the model folder)")
    g.add_argument("--prompt-ids", type=_ids, help="prompt as token ids, e.g. 1,2,3")
    g.add_argument("--max-new-tokens", type=int, default=8)
    g.add_argument("--temperature", type=float, default=0.0, help="0 = greedy")
    g.add_argument("--seed", type=int, default=0, help="sampling seed")
    g.add_argument("--eos-token-id", type=int, action="append", default=None)
    g.add_argument("--block-size", type=int, default=16)

    e = sub.add_parser("engine", help="continuous batching over several requests")
    _add_model_options(e)
    e.add_argument("--block-size", type=int, default=16)
    e.add_argument("--num-blocks", type=int, default=None, help="pages of the cache pool")
    e.add_argument("--kv-memory-fraction", type=float, default=0.8, help="share of free device memory for pages when --num-blocks is not given")
    e.add_argument("--check-cache-visibility", action="store_true", help="debug: refuse reads of pending tokens before their write")
    e.add_argument("--max-running-requests", type=int, default=3)
    e.add_argument("--max-batch-tokens", type=int, default=64)
    e.add_argument("--max-mixed-prefill-tokens", type=int, default=None)
    e.add_argument("--batching-policy", choices=("continuous", "static"), default="continuous")
    e.add_argument("--requests", type=Path, help='JSON list of {"id", "prompt_ids", "max_new_tokens", "arrival_step"}')
    e.add_argument("--num-requests", type=int, default=3, help="synthetic requests when --requests is not given")
    e.add_argument("--prompt-len", type=int, default=9)
    e.add_argument("--max-new-tokens", type=int, default=3)
    e.add_argument("--temperature", type=float, default=0.0)
    e.add_argument("--seed", type=int, default=0)
    e.add_argument("--output-dir", type=Path, help="write result.json and report.md here")

    r = sub.add_parser("random-model", help="write a model folder with random weights")
    r.add_argument("--config", required=True, help="preset name or path to a config.json")
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--out", required=True, type=Path)
    r.add_argument("--storage-dtype", default="bfloat16", choices=("bfloat16", "float32"))
    return parser


def _tokenize(model_dir: Path, text: str) -> list[int]:
    path = model_dir / "tokenizer.json"
    if not path.is_file():
        raise SystemExit(f"--prompt needs {path}; give --prompt-ids instead")
    try:
        from tokenizers import Tokenizer
    except ImportError:
        raise SystemExit("--prompt needs the `tokenizers` package; give --prompt-ids instead") from None
    return Tokenizer.from_file(str(path)).encode(text).ids


def cmd_generate(args: argparse.Namespace) -> int:
    from .config.model_config import read_config_json
    from .engine.config import EngineConfig
    from .engine.factory import default_ops, load_model, make_cache
    from .engine.generation import generate
    from .engine.runner import ModelRunner
    from .sampling.sampler import GREEDY, SamplingParams

    if args.max_new_tokens <= 0:
        raise SystemExit("--max-new-tokens must be > 0")
    if (args.prompt is None) == (args.prompt_ids is None):
        raise SystemExit("give exactly one of --prompt and --prompt-ids")
    prompt = args.prompt_ids if args.prompt_ids is not None else _tokenize(args.model, args.prompt)
    dtype = EngineConfig(dtype=args.dtype).resolved_dtype(read_config_json(args.model))
    ops = default_ops(dtype, "cuda")
    _, model = load_model(args.model, dtype=dtype, device=ops.device)
    need = len(prompt) + args.max_new_tokens
    cache = make_cache(model, block_size=args.block_size, num_blocks=-(-need // args.block_size) + 1, max_requests=1)
    runner = ModelRunner(model, cache, ops)
    sampling = GREEDY if args.temperature == 0 else SamplingParams(args.temperature, args.seed)
    out = generate(
        runner, prompt, max_new_tokens=args.max_new_tokens, eos_token_ids=args.eos_token_id, sampling=sampling
    )
    print(json.dumps({
        "prompt_token_ids": prompt,
        "generated_token_ids": list(out.generated_token_ids),
        "stopped_by_eos": out.stopped_by_eos,
        "prefill_tokens": out.prefill_tokens,
        "decode_steps": out.decode_steps,
        "cache_length": out.cache_length,
    }))
    return 0


def _record_step(result, manager) -> dict[str, Any]:
    """Scheduling, releases and the block tables after the step (the reference's
    `record_step`, experiments/continuous_batch_engine_runner.py:76-99)."""
    active = {}
    for rid in manager.request_ids:
        request = manager.get_request(rid)
        active[rid] = {"block_ids": [list(t) for t in request.tables], "token_count": request.num_tokens}
    return {
        "step": result.plan.index,
        "token_count": result.plan.token_count,
        "prefill": list(result.plan.prompt_ids),
        "decode": list(result.plan.decode_ids),
        "emitted": [list(t) for t in result.report.emitted],
        "finished": list(result.report.finished),
        "released_blocks": {rid: {str(g): list(ids) for g, ids in blocks.items()} for rid, blocks in result.released_blocks},
        "active_cache_after_step": active,
        "cache_stats_after_step": [asdict(s) for s in manager.stats()],
        "step_ms": (result.completed_ns - result.started_ns) / 1e6,
    }


def cmd_engine(args: argparse.Namespace) -> int:
    import torch

    from .engine.config import EngineConfig
    from .engine.engine import ContinuousBatchEngine
    from .engine.scheduler import BatchingPolicy

    config = EngineConfig(
        dtype=args.dtype,
        block_size=args.block_size,
        num_blocks=args.num_blocks,
        kv_memory_fraction=args.kv_memory_fraction,
        max_running_requests=args.max_running_requests,
        max_batch_tokens=args.max_batch_tokens,
        max_mixed_prefill_tokens=args.max_mixed_prefill_tokens,
        batching_policy=BatchingPolicy(args.batching_policy),
        check_cache_visibility=args.check_cache_visibility,
    )
    engine = ContinuousBatchEngine.from_model_dir(args.model, config)
    vocab = engine.runner.vocab_size
    if args.requests is not None:
        requests = json.loads(args.requests.read_text())
    else:
        g = torch.Generator().manual_seed(args.seed)
        requests = [
            {
                "id": chr(ord("A") + i) if i < 26 else f"R{i}",
                "prompt_ids": torch.randint(0, vocab, (max(1, args.prompt_len - 2 * i),), generator=g).tolist(),
                "max_new_tokens": max(1, args.max_new_tokens - i % 3),
                "arrival_step": 0 if i < 2 else i - 1,
            }
            for i in range(args.num_requests)
        ]
    pending = sorted(requests, key=lambda r: r.get("arrival_step", 0))
    records = []
    step_no = 0
    while pending or engine.scheduler.busy:
        while pending and pending[0].get("arrival_step", 0) <= step_no:
            r = pending.pop(0)
            engine.submit(
                str(r["id"]), r["prompt_ids"], max_new_tokens=int(r["max_new_tokens"]),
                eos_token_ids=r.get("eos_token_ids"), temperature=float(r.get("temperature", args.temperature)),
                seed=int(r.get("seed", args.seed)),
            )
        result = engine.step()
        step_no += 1
        if result is None:
            if pending:
                continue
            raise SystemExit("requests are unfinished but the page budget admits no progress")
        records.append(_record_step(result, engine.manager))
        rec = records[-1]
        print(f"step={rec['step']} prefill={rec['prefill']} decode={rec['decode']} finished={rec['finished']}")
    tokens = {str(r["id"]): list(engine.request(str(r["id"])).output) for r in requests}
    all_released = engine.manager.request_ids == () and all(
        g.allocator.free_count == g.num_blocks for g in engine.manager.groups
    )
    metrics = {}
    for rid in tokens:
        m = engine.times(rid)
        metrics[rid] = {"queue_wait_ms": m.queue_wait_ms, "ttft_ms": m.ttft_ms, "median_tpot_ms": m.median_tpot_ms, "e2e_ms": m.e2e_ms}
    for rid, ids in tokens.items():
        print(f"{rid}: ids={ids}")
    print(f"all KV blocks released = {all_released}")
    artifact = {
        "schema_version": 1,
        "artifact": "continuous_batching_run",
        "model": str(args.model),
        "dtype": str(engine.runner.dtype).replace("torch.", ""),
        "block_size": args.block_size,
        "num_blocks": engine.manager.groups[0].num_blocks if engine.manager.groups else 0,
        "requests": requests,
        "steps": records,
        "generated_token_ids": tokens,
        "request_metrics": metrics,
        "all_resources_released": all_released,
    }
    if args.output_dir is not None:
        args.output_dir.mkdir(parents=True, exist_ok=True)
        (args.output_dir / "result.json").write_text(json.dumps(artifact, indent=2))
        lines = ["# Continuous batching run", "", f"model: `{args.model}`, dtype {artifact['dtype']}, block size {args.block_size}", ""]
        lines += ["| step | tokens | prefill | decode | finished |", "|---|---|---|---|---|"]
        lines += [f"| {r['step']} | {r['token_count']} | {r['prefill']} | {r['decode']} | {r['finished']} |" for r in records]
        lines += ["", "| request | generated |", "|---|---|"] + [f"| {rid} | {ids} |" for rid, ids in tokens.items()]
        (args.output_dir / "report.md").write_text("\n".join(lines) + "\n")
        print(f"artifact = {args.output_dir}")
    return 0 if all_released else 1


def cmd_random_model(args: argparse.Namespace) -> int:
    from .config.presets import load_preset
    from .models.registry import config_from_dict
    from .weights.random_init import write_random_model

    config = config_from_dict(load_preset(args.config))
    folder = write_random_model(config, args.out, seed=args.seed, storage_dtype=args.storage_dtype)
    print(folder)
    return 0


def main(argv: Optional[Sequence[str]] = None) -> int:
    args = build_parser().parse_args(argv)
    from . import models  # noqa: F401

    return {"generate": cmd_generate, "engine": cmd_engine, "random-model": cmd_random_model}[args.command](args)


if __name__ == "__main__":
    sys.exit(main())
