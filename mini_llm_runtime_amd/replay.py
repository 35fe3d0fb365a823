"""Trace replay: feed given token ids through a model step by step and write the
logits.  Nothing is sampled.  It drives the framework's own model, step function,
cache manager and kernels, the ones generation uses; it has no forward pass,
cache or loader of its own.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N
                  [--block-size 16] [--max-live 8] [--layers]

Steps come on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

All entries of a step are one batch.  For a step in which something is wanted,
`<out>/<step>.f32` receives the logits at the wanted places, in the order of the
entries and of `want`, as little-endian float32 [wanted, vocab].  After every step
a line `done <step>` is printed and flushed.  With `--layers`, `<out>/<step>.layers.f32`
also receives the residual stream after every execution site at the same places, float32
[sites, wanted, hidden]: where a wrong logit first appears.

The reference's nearest tools capture per-step logits of one request
(src/mini_llm_runtime/generation.py:84-94, `return_step_logits`) and snapshot block
tables per step (experiments/continuous_batch_engine_runner.py:76-99).
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path
from typing import Any, Optional, Sequence, TextIO


PAGE_TOKENS = 16  # default tokens per page of the replay pool
MAX_LIVE = 8  # default number of request slots


def parse_args(argv: Optional[Sequence[str]] = None) -> argparse.Namespace:
    p = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    p.add_argument("--model", required=True, type=Path, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", required=True, choices=("bfloat16", "float32"))
    p.add_argument("--out", required=True, type=Path, help="folder for <step>.f32 files")
    p.add_argument("--max-tokens", required=True, type=int, help="most tokens live requests hold at any time")
    p.add_argument("--block-size", type=int, default=PAGE_TOKENS, help="tokens per page of the cache pool")
    p.add_argument("--max-live", type=int, default=MAX_LIVE, help="most requests that are live at one time")
    p.add_argument("--layers", action="store_true", help="also write <step>.layers.f32: the stream after every site")
    return p.parse_args(argv)


class TraceError(ValueError):
    pass


def _parse_step(line: str) -> dict[str, Any]:
    try:
        step = json.loads(line)
    except json.JSONDecodeError as e:
        raise TraceError(f"not JSON: {e}") from None
    if not isinstance(step, dict) or "step" not in step or "entries" not in step:
        raise TraceError("a step needs the keys 'step' and 'entries'")
    entries = step["entries"]
    if not isinstance(entries, list):
        raise TraceError("'entries' must be a list")
    for e in entries:
        if not isinstance(e, dict) or "id" not in e or "tokens" not in e:
            raise TraceError("an entry needs the keys 'id' and 'tokens'")
        if not isinstance(e["tokens"], list) or not e["tokens"]:
            raise TraceError(f"entry {e.get('id')!r}: 'tokens' must be a non-empty list")
        e.setdefault("want", [])
    step.setdefault("end", [])
    return step


def replay(runner, cache, lines: TextIO, out_dir: Path, done: TextIO, layers: bool = False) -> int:
    """Run every step read from `lines`; returns the number of steps."""
    from .engine.runner import StepEntry

    out_dir.mkdir(parents=True, exist_ok=True)
    count = 0
    for raw in lines:
        raw = raw.strip()
        if not raw:
            continue
        step = _parse_step(raw)
        index = step["step"]
        entries = []
        created = []
        try:
            for e in step["entries"]:
                rid = str(e["id"])
                if not cache.has_request(rid):
                    if cache.slots.free_count == 0:
                        raise TraceError(
                            f"step {index}: request {rid!r} would be live request number "
                            f"{cache.max_requests + 1}; --max-live is {cache.max_requests}"
                        )
                    cache.create_request(rid)
                    created.append(rid)
                entries.append(StepEntry.of(rid, e["tokens"], e["want"]))
            if entries:
                result = runner.step(entries, borrow_logits=True, capture_sites=layers)  # copied out right here
                if result.logits is not None:
                    rows = result.logits.float().cpu().numpy().astype("<f4", copy=False)
                    rows.tofile(out_dir / f"{index}.f32")
                if result.site_outputs is not None:
                    result.site_outputs.float().cpu().numpy().astype("<f4", copy=False).tofile(
                        out_dir / f"{index}.layers.f32"
                    )
        except Exception:
            for rid in created:
                cache.release_request(rid)
            raise
        for rid in step["end"]:
            rid = str(rid)
            if cache.has_request(rid):
                cache.release_request(rid)
        count += 1
        print(f"done {index}", file=done, flush=True)
    return count


def main(argv: Optional[Sequence[str]] = None) -> int:
    args = parse_args(argv)
    if args.max_tokens <= 0 or args.block_size <= 0 or args.max_live <= 0:
        print("trace_run: --max-tokens, --block-size and --max-live must be > 0", file=sys.stderr)
        return 2
    import torch

    from . import models  # noqa: F401  (registers the architectures)
    from .engine.factory import default_ops, load_model, make_cache, parse_dtype
    from .engine.runner import ModelRunner

    dtype = parse_dtype(args.dtype)
    device = torch.device("cuda", 0)
    ops = default_ops(dtype, device)
    _, model = load_model(args.model, dtype=dtype, device=device)
    # the caller rounds every request up to max(64, page) tokens, so whole pages always suffice
    pages = -(-args.max_tokens // args.block_size)
    cache = make_cache(model, block_size=args.block_size, num_blocks=pages, max_requests=args.max_live)
    runner = ModelRunner(model, cache, ops)
    try:
        replay(runner, cache, sys.stdin, args.out, sys.stdout, layers=args.layers)
    except Exception as e:  # a bad trace or a failed step ends the run with a message
        print(f"trace_run: {type(e).__name__}: {e}", file=sys.stderr)
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())
