"""Decode and prefill throughput of the engine on one MI355X, random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config qwen2.5-0.5b] [--layers L]

Default run: the Qwen2.5-0.5B shape in bfloat16, 8 requests with 2,048-token
random-id prompts (context capacity 4,096, KV block 16).  A step is one decode
step of the whole continuous-batching engine: scheduling, the step function over
the batch, sampling on the GPU and the copy of the chosen tokens to the host.  W warm-up steps, then exactly K
timed steps between device synchronisations.  One JSON line is printed:
`value` is decoded tokens per second at batch 8; `points` holds batch 1 and 64;
`prefill` is one 2,048-token prompt; `roofline` prices the decode step by the
bytes it must read (every weight once and the live requests' cache) against
8 TB/s.  Peaks are MI355X's published dense figures.
"""

from __future__ import annotations

import argparse
import json
import sys
import tempfile
import time
from pathlib import Path

HBM_BYTES_PER_S = 8.0e12
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
PROMPT_LEN = 2048
CONTEXT_LEN = 4096
BLOCK_SIZE = 16


def parse_args() -> argparse.Namespace:
    p = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=64)
    p.add_argument("--warmup", type=int, default=8)
    p.add_argument("--config", default="qwen2.5-0.5b", help="preset name or path to a config.json")
    p.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    p.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    p.add_argument("--batch", type=int, default=8)
    p.add_argument("--points", default="1,64", help="further decode batch sizes, comma separated ('' for none)")
    p.add_argument("--prompt-len", type=int, default=PROMPT_LEN)
    p.add_argument("--no-prefill", action="store_true", help="skip the prefill measurement")
    p.add_argument("--seed", type=int, default=0)
    return p.parse_args()


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported", flush=True)
        return 2

    import torch

    sys.path.insert(0, str(Path(__file__).resolve().parent))
    import mini_llm_runtime_amd  # noqa: F401
    from mini_llm_runtime_amd.config.presets import load_preset
    from mini_llm_runtime_amd.engine.factory import default_ops, load_model, make_cache, parse_dtype
    from mini_llm_runtime_amd.engine import ContinuousBatchEngine, PagedBlockAdmissionController, RequestScheduler
    from mini_llm_runtime_amd.engine.runner import ModelRunner, StepEntry
    from mini_llm_runtime_amd.models.registry import config_from_dict
    from mini_llm_runtime_amd.sampling.sampler import Sampler
    from mini_llm_runtime_amd.weights.random_init import write_random_model

    data = load_preset(args.config)
    full_layers = int(data["num_hidden_layers"])
    if args.layers is not None:
        data["num_hidden_layers"] = int(args.layers)
    config = config_from_dict(data)
    dtype = parse_dtype(args.dtype)
    short = "bf16" if dtype == torch.bfloat16 else "fp32"
    device = torch.device("cuda", 0)
    ops = default_ops(dtype, device)

    with tempfile.TemporaryDirectory(prefix="mlr_bench_") as tmp:
        folder = write_random_model(config, tmp, seed=args.seed, storage_dtype="bfloat16")
        _, model = load_model(folder, dtype=dtype, device=device)

    batches = [args.batch] + [int(b) for b in args.points.split(",") if b.strip()]
    steps_total = args.warmup + args.steps
    capacity = max(CONTEXT_LEN, args.prompt_len + steps_total + max(batches) + 9)
    pages = max(batches) * (-(-capacity // BLOCK_SIZE)) + 8
    cache = make_cache(model, block_size=BLOCK_SIZE, num_blocks=pages, max_requests=max(batches))
    runner = ModelRunner(model, cache, ops)
    sampler = Sampler(ops, device)
    vocab = config.vocab_size
    gen = torch.Generator().manual_seed(args.seed)

    def prompt() -> list[int]:
        return torch.randint(0, vocab, (args.prompt_len,), generator=gen).tolist()

    def sync() -> None:
        torch.cuda.synchronize(device)

    def decode(batch: int, warmup: int, steps: int) -> float:
        """ms per decode step of the continuous-batching engine at this batch size, contexts
        starting at prompt_len: scheduler, step function, sampling on the GPU, tokens to the host."""
        admission = PagedBlockAdmissionController(cache, max_step_tokens=args.prompt_len)
        scheduler = RequestScheduler(
            max_running_requests=batch,
            max_batch_tokens=max(args.prompt_len, batch),
            admission_callback=admission.try_admit,
        )
        engine = ContinuousBatchEngine(scheduler=scheduler, runner=runner, admission=admission, sampler=sampler)
        for i in range(batch):
            engine.submit(f"b{batch}-{i}", prompt(), max_new_tokens=warmup + steps + batch + 8)
        while True:  # prompts, until a step is nothing but one token for every request
            result = engine.step()
            if len(result.batch.decode_request_ids) == batch:
                break
        for _ in range(warmup):
            engine.step()
        sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            result = engine.step()
        sync()
        elapsed = time.perf_counter() - t0
        assert len(result.batch.decode_request_ids) == batch and len(result.update.emitted_tokens) == batch
        engine.run_until_done()
        return elapsed * 1e3 / steps

    from mini_llm_runtime_amd.sampling.sampler import GREEDY as _GREEDY

    ms_main = decode(args.batch, args.warmup, args.steps)
    value = args.batch * 1e3 / ms_main
    points = {}
    for b in batches[1:]:
        ms = decode(b, max(2, args.warmup // 2), max(8, args.steps // 2))
        points[f"decode_b{b}"] = round(b * 1e3 / ms, 1)

    # ---- what a decode step has to read ------------------------------------------------------
    weight_bytes = model.weight_bytes()
    embed_bytes = model.embed_weight.numel() * model.embed_weight.element_size()
    if not config.tie_word_embeddings:
        weight_bytes -= embed_bytes  # an untied input table is only gathered from
    kv_per_token = sum(
        2 * len(g.sites) * g.spec.num_kv_heads * g.spec.head_dim * g.key.element_size() for g in cache.groups
    )
    mean_context = args.prompt_len + args.warmup + args.steps / 2
    step_bytes = weight_bytes + args.batch * mean_context * kv_per_token
    achieved = step_bytes / (ms_main * 1e-3)
    roofline = {
        "bound": "hbm",
        "achieved": round(achieved / 1e9, 1),
        "peak": HBM_BYTES_PER_S / 1e9,
        "unit": "GB/s",
        "frac": round(achieved / HBM_BYTES_PER_S, 4),
    }

    # ---- prefill of one prompt ----------------------------------------------------------------
    prefill = None
    if not args.no_prefill:
        tokens = args.prompt_len
        times = []
        for i in range(5):
            rid = f"p{i}"
            cache.create_request(rid)
            entry = [StepEntry.of(rid, prompt(), (tokens - 1,))]
            sync()
            t0 = time.perf_counter()
            out = runner.step(entry)
            sampler.sample(out.logits, [_GREEDY], [0]).cpu()
            sync()
            times.append(time.perf_counter() - t0)
            cache.release_request(rid)
        ms = sorted(times[1:])[len(times[1:]) // 2] * 1e3
        d = config.head_dim
        per_layer = (
            config.hidden_size * (config.num_attention_heads + 2 * config.num_key_value_heads) * d
            + config.num_attention_heads * d * config.hidden_size
            + 3 * config.hidden_size * config.intermediate_size
        )
        flops = (
            2 * tokens * per_layer * config.num_hidden_layers
            + config.num_hidden_layers * config.num_attention_heads * 4 * d * tokens * (tokens + 1) // 2
            + 2 * config.vocab_size * config.hidden_size
        )
        prefill = {
            "value": round(tokens * 1e3 / ms, 1),
            "tokens": tokens,
            "ms": round(ms, 3),
            "frac": round(flops / (ms * 1e-3) / PEAK_FLOPS[short], 4),
        }

    line = {
        "metric": "decode tokens/s",
        "value": round(value, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_main, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": short,
        "data": "synthetic (random weights, uniform random token ids)",
        "config": {
            "model": f"{args.config} shape",
            "global_batch": args.batch,
            "seq_len": CONTEXT_LEN,
            "prompt_len": args.prompt_len,
            "parallelism": "single GPU",
            "layers": config.num_hidden_layers,
            "layers_full_model": full_layers,
            "hidden_size": config.hidden_size,
            "num_attention_heads": config.num_attention_heads,
            "num_key_value_heads": config.num_key_value_heads,
            "head_dim": config.head_dim,
            "intermediate_size": config.intermediate_size,
            "vocab_size": config.vocab_size,
            "tie_word_embeddings": config.tie_word_embeddings,
            "kv_block_size": BLOCK_SIZE,
            "weight_bytes": int(weight_bytes),
            "kv_bytes_per_token": int(kv_per_token),
        },
        "prefill": prefill,
        "roofline": roofline,
        "points": points,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
