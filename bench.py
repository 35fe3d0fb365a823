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
8 TB/s.  Peaks are MI355X's published dense figures.  `points_7b` and `points_32b`
(default run only; `--no-large` leaves them out) hold decode at batch 1, 8 and 64 (tokens a
second, step time, share of the HBM bound) and the prefill for the two larger shapes, the
7B shape's burst workload and the 32B shape's chunked workload (below) as `burst` and
`chunked`, with the number of layers run and of the full model beside them;
`points_ctx16k` decode at batch 8 and the prefill at a context of 16,384 tokens for the 0.5B
and the 7B shape, `points_reference` the reference's own published measurements at their parameters
beside its figures (`--workload reference`, below).  `peak_memory_gb` (per shape) is the most device memory the run held.

How it measures (the reference's harness rules, src/mini_llm_runtime/timing.py:49-82,
141-160 and environment.py:37-93): untimed warm-up first; the timed steps between
device synchronisations; the whole timed region also between two device events
(`ms_per_step_device`); every step's host time kept as a raw sample (`samples_ms`,
`median_ms`, `p10_ms`, `p90_ms`; with decoding one step ahead a sample is the time between
two steps' tokens reaching the host); `env` records versions, device, commit and whether the
tree was dirty.  Nothing that compiles or records a graph is timed.

Two further workloads print a JSON line of their own (`--workload`):
`burst`: 64 requests arrive at once, prompt lengths uniform in [128, 2048], 32/64/128/256 new
tokens in turn, 2,048 tokens a step: generated tokens a second, medians of the time to the
first token and of the time between tokens.  `chunked`: 32 requests decode at context 2,048
while one 8,192-token prompt is taken in four portions of 2,048 tokens beside them: the time of
such a mixed step, which is also the time between the decoding requests' tokens.
`library`: where one prompt step's time goes, by entry point of the kernel library (device events
around every call of an untimed extra step), and beside it what the vendor library's routines take
for the same shapes on the same card (torch's linear for the four products of a layer, its
scaled_dot_product_attention for the attention): a yardstick for the hand-written kernels; none of
those routines is on the engine's path.
`reference`: the reference's own published measurements, run here at their parameters with the
0.5B shape (random weights and token ids of the published lengths; its figures are of an RTX 3060
laptop GPU in float16 and stand beside for scale): the burst of 8 short requests under continuous and
static batching (docs/benchmarks/static-continuous.json: prompts of 3/7/4/9 tokens, 2/4/8/12 new
tokens, 4 running requests, 64 tokens a step, block 16, 3 warm-up runs and 10 measured), the time to the
first token of a request that arrives when the first four have reserved all 28 pages or 28 of 29
(scripts/benchmark_block_pressure_ttft.py:25-45, 170-232), the prompt step
of 4 x 512 and of 4 x 256 tokens (docs/benchmarks/prefill-4x512.json, docs/prefill_attention_backends.md:73-77)
and the decode attention at one request and a
context of 2,048 (docs/split_kv_sweep.md:38-46).
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


def long_context_points(args) -> dict:
    """Decode at batch 8 and the prefill at a context of 16,384 tokens, for the 0.5B and the 7B shape."""
    import copy

    long_args = copy.copy(args)
    long_args.prompt_len = 16384
    out = {"context": long_args.prompt_len}
    for tag, name, layers in (("0.5b", "qwen2.5-0.5b", None), ("7b", "qwen2.5-7b", None)):
        point = large_point(long_args, name, layers)
        out[f"decode_b8_{tag}"] = point["decode_b8"]
        out[f"decode_b8_{tag}_hbm_frac"] = point["decode_b8_hbm_frac"]
        if "prefill" in point:
            out[f"prefill_{tag}_ms"] = point["prefill_ms"]
            out[f"prefill_{tag}_frac"] = point["prefill_frac"]
    return out


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
    p.add_argument("--workload", default="decode", choices=("decode", "burst", "chunked", "library", "reference"))
    p.add_argument("--no-large", action="store_true", help="leave out the 7B and 32B points of the default run")
    p.add_argument("--samples", action="store_true", help="print every raw sample, not only their summary")
    p.add_argument("--layers-32b", type=int, default=None, help="layers of the 32B shape's points (default: all 64)")
    p.add_argument("--tuning", default="", help="KernelTuning fields to change, e.g. finish_stream=false,decode_partition=128")
    return p.parse_args()


def kernel_tuning(text: str):
    """A KernelTuning with the fields named in `text` (name=value, comma separated) changed; None for none."""
    from dataclasses import fields, replace

    from mini_llm_runtime_amd.kernels.tuning import KernelTuning

    if not text:
        return None
    kinds = {f.name: f.type for f in fields(KernelTuning)}
    changes = {}
    for item in text.split(","):
        name, _, value = item.partition("=")
        name = name.strip()
        if name not in kinds:
            raise SystemExit(f"--tuning: KernelTuning has no field {name!r} (it has {', '.join(sorted(kinds))})")
        default = getattr(KernelTuning(), name)
        changes[name] = value.strip().lower() in ("1", "true", "yes", "on") if isinstance(default, bool) else int(value)
    return replace(KernelTuning(), **changes)


def median(values):
    ordered = sorted(values)
    return ordered[len(ordered) // 2]


def workload_config(args, config, full_layers: int) -> dict:
    return {
        "model": f"{args.config} shape",
        "layers": config.num_hidden_layers,
        "layers_full_model": full_layers,
        "hidden_size": config.hidden_size,
        "num_attention_heads": config.num_attention_heads,
        "num_key_value_heads": config.num_key_value_heads,
        "head_dim": config.head_dim,
        "intermediate_size": config.intermediate_size,
        "vocab_size": config.vocab_size,
        "kv_block_size": BLOCK_SIZE,
    }


def burst(args, config, full_layers, model, ops, device) -> dict:
    """64 requests at once through the continuous-batching engine, 2,048 tokens a step."""
    import random

    import torch

    from mini_llm_runtime_amd.engine import ContinuousBatchEngine, PageAdmission, Scheduler
    from mini_llm_runtime_amd.engine.factory import make_cache
    from mini_llm_runtime_amd.engine.runner import ModelRunner
    from mini_llm_runtime_amd.sampling.sampler import Sampler

    requests, budget = 64, 2048
    pages = requests * (-(-(2048 + 256) // BLOCK_SIZE)) + 8
    cache = make_cache(model, block_size=BLOCK_SIZE, num_blocks=pages, max_requests=requests)
    runner = ModelRunner(model, cache, ops)
    sampler = Sampler(ops, device)

    def run(seed: int):
        admission = PageAdmission(cache, max_step_tokens=budget)
        scheduler = Scheduler(
            max_running_requests=requests, max_batch_tokens=budget, admit=admission.admit
        )
        engine = ContinuousBatchEngine(scheduler=scheduler, runner=runner, admission=admission, sampler=sampler)
        rng = random.Random(seed)
        prompt_tokens = generated = 0
        torch.cuda.synchronize(device)
        t0 = time.perf_counter()
        for i in range(requests):
            n, new = rng.randint(128, 2048), (32, 64, 128, 256)[i % 4]
            engine.submit(f"s{seed}-{i}", [rng.randrange(config.vocab_size) for _ in range(n)], max_new_tokens=new)
            prompt_tokens += n
            generated += new
        steps = 0
        while engine.scheduler.busy:
            engine.step()
            steps += 1
        torch.cuda.synchronize(device)
        seconds = time.perf_counter() - t0
        shots = engine.all_times()
        return {
            "seconds": seconds,
            "steps": steps,
            "prompt_tokens": prompt_tokens,
            "generated": generated,
            "ttft_ms": median([m.ttft_ms for m in shots]),
            "tpot_ms": median([m.median_tpot_ms for m in shots]),
        }

    if args.warmup:
        run(args.seed + 1000)  # libraries loaded, the decode steps' graphs recorded
    runs = [run(args.seed + r) for r in range(3)]
    best = median([(r["seconds"], i) for i, r in enumerate(runs)])[1]
    r = runs[best]
    return {
        "metric": "burst generated tokens/s",
        "value": round(r["generated"] / r["seconds"], 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "higher_is_better": True,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic (random weights, uniform random token ids)",
        "seconds": round(r["seconds"], 4),
        "engine_steps": r["steps"],
        "prompt_tokens": r["prompt_tokens"],
        "generated_tokens": r["generated"],
        "total_tokens_per_s": round((r["prompt_tokens"] + r["generated"]) / r["seconds"], 1),
        "median_ttft_ms": round(r["ttft_ms"], 2),
        "median_tpot_ms": round(r["tpot_ms"], 3),
        "runs_seconds": [round(x["seconds"], 4) for x in runs],
        "config": dict(workload_config(args, config, full_layers), requests=requests, max_batch_tokens=budget),
    }


def chunked(args, config, full_layers, model, ops, device) -> dict:
    """One 8,192-token prompt in portions of 2,048 tokens beside 32 decoding requests."""
    import torch

    from mini_llm_runtime_amd.engine import ContinuousBatchEngine, PageAdmission, Scheduler
    from mini_llm_runtime_amd.engine.factory import make_cache
    from mini_llm_runtime_amd.engine.runner import ModelRunner
    from mini_llm_runtime_amd.sampling.sampler import Sampler

    decoders, context, long_prompt, portion, repeats = 32, 2048, 8192, 2048, 3
    new_tokens = decoders + 64 + (repeats + 2) * (long_prompt // portion + 2)
    pages = decoders * (-(-(context + new_tokens) // BLOCK_SIZE)) + (long_prompt + 16) // BLOCK_SIZE + 8
    cache = make_cache(model, block_size=BLOCK_SIZE, num_blocks=pages, max_requests=decoders + 1)
    runner = ModelRunner(model, cache, ops)
    sampler = Sampler(ops, device)
    admission = PageAdmission(cache, max_step_tokens=portion + decoders)
    scheduler = Scheduler(
        max_running_requests=decoders + 1,
        max_batch_tokens=portion + decoders,
        max_mixed_prefill_tokens=portion,
        admit=admission.admit,
    )
    engine = ContinuousBatchEngine(scheduler=scheduler, runner=runner, admission=admission, sampler=sampler)
    gen = torch.Generator().manual_seed(args.seed)

    def ids(n: int) -> list[int]:
        return torch.randint(0, config.vocab_size, (n,), generator=gen).tolist()

    def timed_step():
        torch.cuda.synchronize(device)
        t0 = time.perf_counter()
        result = engine.step()
        torch.cuda.synchronize(device)
        return result, (time.perf_counter() - t0) * 1e3

    for i in range(decoders):
        engine.submit(f"d{i}", ids(context), max_new_tokens=new_tokens)
    while len(engine.step().plan.decode_ids) < decoders:
        pass
    for _ in range(8):
        engine.step()
    alone = median([timed_step()[1] for _ in range(16)])
    portions = long_prompt // portion
    warmups = 2  # a shape of step is run plainly when it first comes and recorded when it comes again
    mixed = [[] for _ in range(portions)]
    behind = []
    for r in range(warmups + repeats):
        engine.submit(f"long{r}", ids(long_prompt), max_new_tokens=1)
        for i in range(portions):
            result, ms = timed_step()
            batch = result.plan
            assert batch.prompt_ids == (f"long{r}",) and len(batch.decode_ids) == decoders
            assert batch.token_count == portion + decoders
            if r >= warmups:
                mixed[i].append(ms)
        result, ms = timed_step()
        assert not result.plan.prompt_ids
        if r >= warmups:
            behind.append(ms)
    by_portion = [median(times) for times in mixed]
    # The engine launches a decode step ahead whenever the next step is known to be one.  The step of
    # the last portion therefore launches the decode step behind it before it returns, and that one
    # launches another (which the next prompt's arrival then discards); the waits of this loop at
    # the end of both steps cover a decode step each that is no part of the portion.
    by_portion[-1] += median(behind) - 2 * alone
    ms = sum(by_portion) / portions
    return {
        "metric": "mixed step: 2,048 prompt tokens beside 32 decoding requests (mean over the prompt's portions)",
        "value": round(ms, 3),
        "unit": "ms",
        "n_gpus": 1,
        "higher_is_better": False,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic (random weights, uniform random token ids)",
        "decoders_tpot_ms_beside_the_prompt": round(ms, 3),
        "decoders_tpot_ms_alone": round(alone, 3),
        "prompt_tokens_per_s": round(portion * 1e3 / ms, 1),
        "mixed_steps_ms_by_portion": [round(x, 3) for x in by_portion],
        "decode_step_behind_the_prompt_ms": round(median(behind), 3),
        "config": dict(
            workload_config(args, config, full_layers),
            decoders=decoders,
            decoders_context=context,
            prompt_len=long_prompt,
            portion=portion,
        ),
    }


def reference_measurements(args, bench) -> dict:
    """The reference's three published measurements at their own parameters (see the module's text)."""
    import random
    from types import SimpleNamespace

    import torch

    from mini_llm_runtime_amd.engine import BatchingPolicy, ContinuousBatchEngine, PageAdmission, Scheduler
    from mini_llm_runtime_amd.engine.factory import make_cache
    from mini_llm_runtime_amd.engine.runner import ModelRunner, StepEntry
    from mini_llm_runtime_amd.sampling.sampler import Sampler

    config, model, ops, device = bench.config, bench.model, bench.ops, bench.device
    published = {
        "continuous": {"tokens_per_s": 71.70, "median_ttft_ms": 178.08, "median_tpot_ms": 25.56, "median_e2e_ms": 414.06},
        "static": {"tokens_per_s": 65.43, "median_ttft_ms": 334.78, "median_tpot_ms": 24.06, "median_e2e_ms": 478.58},
        "late_request_ttft_ms": {"28_blocks": 76.73, "29_blocks": 52.46, "paired_difference": 23.60},
        "prefill_4x512_ms": 136.475,
        "prefill_4x256_ms": 68.77,
        "decode_attention_us": 77.0,
        "hardware": "RTX 3060 Laptop, float16 (README.md:79-95, 114-115; docs/split_kv_sweep.md:38-46; docs/block_pressure_ttft_benchmark.md:38-41; docs/prefill_attention_backends.md:73-77)",
    }
    # 1. the burst of 8 short requests, both policies
    specs = [(3, 2), (7, 4), (4, 8), (9, 12)] * 2
    cache = make_cache(model, block_size=16, num_blocks=64, max_requests=4)
    runner = ModelRunner(model, cache, ops)
    sampler = Sampler(ops, device)

    def burst_of_eight(policy, seed: int) -> dict:
        admission = PageAdmission(cache, max_step_tokens=64)
        scheduler = Scheduler(max_running_requests=4, max_batch_tokens=64, admit=admission.admit, batching_policy=policy)
        engine = ContinuousBatchEngine(scheduler=scheduler, runner=runner, admission=admission, sampler=sampler)
        rng = random.Random(seed)
        torch.cuda.synchronize(device)
        begin = time.perf_counter()
        for i, (prompt, new) in enumerate(specs):
            engine.submit(f"r{i}", [rng.randrange(config.vocab_size) for _ in range(prompt)], max_new_tokens=new)
        while engine.scheduler.busy:
            engine.step()
        torch.cuda.synchronize(device)
        seconds = time.perf_counter() - begin
        shots = engine.all_times()
        return {
            "tokens_per_s": sum(new for _, new in specs) / seconds,
            "median_ttft_ms": median([t.ttft_ms for t in shots]),
            "median_tpot_ms": median([t.median_tpot_ms for t in shots if t.median_tpot_ms is not None]),
            "median_e2e_ms": median([t.e2e_ms for t in shots]),
        }

    policies = {"continuous": BatchingPolicy.CONTINUOUS, "static": BatchingPolicy.STATIC}
    samples = {name: [] for name in policies}
    for trial in range(3 + 10):  # the cases take turns, in reversed order on odd rounds, as published
        order = list(policies) if trial % 2 == 0 else list(policies)[::-1]
        for name in order:
            shot = burst_of_eight(policies[name], args.seed)
            if trial >= 3:
                samples[name].append(shot)
    bursts = {
        name: {key: round(median([shot[key] for shot in shots]), 3) for key in shots[0]} for name, shots in samples.items()
    }
    del runner, cache
    # 1b. a request that arrives behind step 0 when the first four have reserved every page (28) or all but one (29)
    first, late = [(128, 2), (128, 3), (128, 3), (1, 3)], (7, 2)
    pools = {}
    for blocks in (28, 29):
        pool = make_cache(model, block_size=16, num_blocks=blocks, max_requests=5)
        pools[blocks] = (pool, ModelRunner(model, pool, ops))

    def late_arrival(blocks: int) -> dict:
        pool, pool_runner = pools[blocks]
        admission = PageAdmission(pool, max_step_tokens=sum(n for n, _ in first))
        scheduler = Scheduler(max_running_requests=5, max_batch_tokens=sum(n for n, _ in first), admit=admission.admit)
        engine = ContinuousBatchEngine(scheduler=scheduler, runner=pool_runner, admission=admission, sampler=sampler)
        rng = random.Random(args.seed)
        for i, (prompt, new) in enumerate(first):
            engine.submit(f"first{i}", [rng.randrange(config.vocab_size) for _ in range(prompt)], max_new_tokens=new)
        engine.step()
        engine.submit("late", [rng.randrange(config.vocab_size) for _ in range(late[0])], max_new_tokens=late[1])
        while engine.scheduler.busy:
            engine.step()
        shot = engine.times("late")
        return {"ttft_ms": shot.ttft_ms, "queue_wait_ms": shot.queue_wait_ms}

    waits = {28: [], 29: []}
    for trial in range(3 + 10):
        for blocks in ((28, 29) if trial % 2 == 0 else (29, 28)):
            shot = late_arrival(blocks)
            if trial >= 3:
                waits[blocks].append(shot)
    late_request = {
        f"{blocks}_blocks": {key: round(median([shot[key] for shot in shots]), 3) for key in shots[0]}
        for blocks, shots in waits.items()
    }
    late_request["paired_ttft_difference_ms"] = round(
        median([a["ttft_ms"] - b["ttft_ms"] for a, b in zip(waits[28], waits[29])]), 3)
    del pools
    # 2. four prompts of 512 (and of 256) tokens in one step of the step function (model and cache write only)
    cache = make_cache(model, block_size=16, num_blocks=4 * 32 + 8, max_requests=4)
    runner = ModelRunner(model, cache, ops)
    gen = torch.Generator().manual_seed(args.seed)
    prefill_of_four = {}
    for length in (512, 256):
        times = []
        for trial in range(2 + 6):
            entries = []
            for i in range(4):
                cache.create_request(f"p{i}")
                ids = torch.randint(0, config.vocab_size, (length,), generator=gen).tolist()
                entries.append(StepEntry.of(f"p{i}", ids, (length - 1,)))
            torch.cuda.synchronize(device)
            begin = time.perf_counter()
            runner.step(entries, borrow_logits=True)
            torch.cuda.synchronize(device)
            times.append((time.perf_counter() - begin) * 1e3)
            for i in range(4):
                cache.release_request(f"p{i}")
        prefill_of_four[length] = median(times[2:])
    prefill_ms = prefill_of_four[512]
    del runner, cache
    # 3. the decode attention alone: one request, context 2,048, on the cache's page layout
    heads, kv, d, bs, ctx_len = config.num_attention_heads, config.num_key_value_heads, config.head_dim, 16, 2048
    pages = ctx_len // bs
    g = torch.Generator(device=device).manual_seed(args.seed)
    rand = lambda *shape: torch.randn(*shape, device=device, generator=g).to(bench.dtype)  # noqa: E731
    key_pages, value_pages, q = rand(pages, kv, bs, d), rand(pages, kv, d, bs), rand(1, heads * d)
    table = torch.randperm(pages, device=device).to(torch.int32).view(1, pages)
    one = lambda v: torch.tensor(v, dtype=torch.int32, device=device)  # noqa: E731
    plan = SimpleNamespace(num_entries=1, token_entry=one([0]), positions=one([ctx_len - 1]), cu_q=one([0, 1]),
                           context_lens=one([ctx_len]), max_context_len=ctx_len, max_q_len=1, num_query_tiles=0,
                           num_decode_entries=1, max_decode_context=ctx_len)
    attend = lambda: ops.paged_attention(  # noqa: E731
        q, key_pages, value_pages, table, plan, plan=plan, num_heads=heads, num_kv_heads=kv, head_dim=d, block_size=bs,
        scale=d ** -0.5, window=None)
    for _ in range(3):
        attend()
    torch.cuda.synchronize(device)
    graph, kept = torch.cuda.CUDAGraph(), []  # 50 calls recorded and replayed: the kernels' time, not the host's
    with torch.inference_mode(), torch.cuda.graph(graph):  # (as the engine records its steps)
        for _ in range(50):
            kept.append(attend())
    graph.replay()
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize(device)
    begin.record()
    for _ in range(10):
        graph.replay()
    end.record()
    torch.cuda.synchronize(device)
    attention_us = begin.elapsed_time(end) * 1e3 / 500
    return {
        "metric": "the reference's published measurements at their own parameters",
        "value": bursts["continuous"]["tokens_per_s"],
        "unit": "tokens/s (continuous batching, burst of 8 short requests)",
        "n_gpus": 1,
        "higher_is_better": True,
        "vs_baseline": round(bursts["continuous"]["tokens_per_s"] / published["continuous"]["tokens_per_s"], 1),
        "dtype": bench.short,
        "data": "synthetic (random weights, uniform random token ids of the published lengths)",
        "burst_of_8": bursts,
        "late_request_under_page_pressure": late_request,
        "prefill_4x512_ms": round(prefill_ms, 3),
        "prefill_4x256_ms": round(prefill_of_four[256], 3),
        "decode_attention_us": round(attention_us, 2),
        "published": published,
        "config": dict(workload_config(args, config, bench.full_layers), requests=8, max_running_requests=4,
                       max_batch_tokens=64, kv_block_size=16),
    }


def library_yardstick(args, bench) -> dict:
    """One prompt step with device events around every call into the kernel library, summed by entry
    point (products by their weight's shape), and the vendor library's time for the layer's four
    products and its attention at the same sizes."""
    import torch
    import torch.nn.functional as F

    from mini_llm_runtime_amd.engine.runner import StepEntry

    config, tokens, device = bench.config, args.prompt_len, bench.device
    layers = config.num_hidden_layers
    events = []
    plain_call = bench.ops._call

    def timed_call(name, *call_args, lib=None):
        label = name
        if name == "mlr_gemm_bf16":
            label = f"{name} n={call_args[10]} k={call_args[11]}" + (" swiglu" if call_args[6] else "")
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        plain_call(name, *call_args, lib=lib)
        end.record()
        events.append((label, begin, end))

    def step(rid):
        bench.cache.create_request(rid)
        bench.runner.step([StepEntry.of(rid, bench.prompt(), (tokens - 1,))], borrow_logits=True)
        bench.sync()
        bench.cache.release_request(rid)

    bench.runner.use_graphs = False  # events cannot be recorded into a graph
    step("warm")
    bench.ops._call = timed_call
    try:
        step("timed")
    finally:
        bench.ops._call = plain_call
    entry_points = {}
    for label, begin, end in events:
        row = entry_points.setdefault(label, {"calls": 0, "us": 0.0})
        row["calls"] += 1
        row["us"] += begin.elapsed_time(end) * 1e3
    for row in entry_points.values():
        row["us"] = round(row["us"], 1)
        row["us_per_call"] = round(row["us"] / row["calls"], 1)

    def timed(fn, repeats=10):
        for _ in range(3):
            fn()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        bench.sync()
        begin.record()
        for _ in range(repeats):
            fn()
        end.record()
        bench.sync()
        return round(begin.elapsed_time(end) * 1e3 / repeats, 1)

    gen = torch.Generator(device=device).manual_seed(args.seed)
    rand = lambda *shape: (torch.randn(*shape, device=device, generator=gen) * 0.05).to(bench.dtype)  # noqa: E731
    d, heads, kv = config.head_dim, config.num_attention_heads, config.num_key_value_heads
    hidden, inter = config.hidden_size, config.intermediate_size
    library = {}
    for name, n, k in (("qkv", (heads + 2 * kv) * d, hidden), ("o", hidden, heads * d), ("gate_up", 2 * inter, hidden),
                       ("down", hidden, inter)):
        x, w = rand(tokens, k), rand(n, k)
        library[f"linear_{name} n={n} k={k}"] = timed(lambda: F.linear(x, w))
        del x, w
    q, key, value = rand(1, heads, tokens, d), rand(1, heads, tokens, d), rand(1, heads, tokens, d)
    library["scaled_dot_product_attention causal"] = timed(lambda: F.scaled_dot_product_attention(q, key, value, is_causal=True))
    return {
        "metric": "prompt step by entry point, and the vendor library's routines at the same sizes",
        "unit": "us",
        "n_gpus": 1,
        "dtype": bench.short,
        "config": {"model": f"{args.config} shape", "layers": layers, "prompt_len": tokens, "hidden_size": hidden,
                   "intermediate_size": inter, "num_attention_heads": heads, "num_key_value_heads": kv, "head_dim": d},
        "entry_points": dict(sorted(entry_points.items(), key=lambda item: -item[1]["us"])),
        "library_us_per_call": library,
    }


def environment() -> dict:
    """What the numbers were measured on (src/mini_llm_runtime/environment.py:37-93 of the
    reference records the same kinds of facts)."""
    import platform
    import subprocess

    import torch

    root = Path(__file__).resolve().parent

    def git(*args: str) -> str:
        try:
            return subprocess.run(["git", *args], cwd=root, capture_output=True, text=True, timeout=10).stdout.strip()
        except (OSError, subprocess.SubprocessError):
            return ""

    props = torch.cuda.get_device_properties(0)
    return {
        "python": platform.python_version(),
        "torch": torch.__version__,
        "hip": torch.version.hip,
        "device": props.name,
        "arch": getattr(props, "gcnArchName", ""),
        "compute_units": props.multi_processor_count,
        "memory_gb": round(props.total_memory / 2**30, 1),
        "commit": git("rev-parse", "--short", "HEAD") or None,
        "dirty": bool(git("status", "--porcelain", "--untracked-files=no")) if git("rev-parse", "HEAD") else None,
    }


def summary(samples_ms: list, keep: bool) -> dict:
    ordered = sorted(samples_ms)
    n = len(ordered)
    out = {
        "count": n,
        "median_ms": round(ordered[n // 2], 4),
        "p10_ms": round(ordered[n // 10], 4),
        "p90_ms": round(ordered[min(n - 1, (9 * n) // 10)], 4),
        "min_ms": round(ordered[0], 4),
        "max_ms": round(ordered[-1], 4),
    }
    if keep:
        out["samples_ms"] = [round(x, 4) for x in samples_ms]
    return out


class Bench:
    """One model shape with random weights on the device, and the measurements on it."""

    def __init__(self, args, name: str, layers, batches: list):
        import torch

        from mini_llm_runtime_amd.config.presets import load_preset
        from mini_llm_runtime_amd.engine.factory import default_ops, make_cache, parse_dtype
        from mini_llm_runtime_amd.engine.runner import ModelRunner
        from mini_llm_runtime_amd.models.registry import build_model, config_from_dict
        from mini_llm_runtime_amd.sampling.sampler import Sampler
        from mini_llm_runtime_amd.weights.random_init import bind_random_weights

        self.args = args
        self.name = name
        data = load_preset(name)
        self.full_layers = int(data["num_hidden_layers"])
        if layers is not None:
            data["num_hidden_layers"] = int(layers)
        self.config = config_from_dict(data)
        self.dtype = parse_dtype(args.dtype)
        self.short = "bf16" if self.dtype == torch.bfloat16 else "fp32"
        self.device = torch.device("cuda", 0)
        self.ops = default_ops(self.dtype, self.device, kernel_tuning(args.tuning))
        self.model = build_model(self.config)
        bind_random_weights(self.model, seed=args.seed, dtype=self.dtype, device=self.device)
        self.batches = batches
        steps_total = args.warmup + args.steps
        capacity = max(CONTEXT_LEN, args.prompt_len + steps_total + max(batches) + 9)
        pages = max(batches) * (-(-capacity // BLOCK_SIZE)) + 8
        self.cache = make_cache(self.model, block_size=BLOCK_SIZE, num_blocks=pages, max_requests=max(batches))
        self.runner = ModelRunner(self.model, self.cache, self.ops)
        self.sampler = Sampler(self.ops, self.device)
        self.gen = torch.Generator().manual_seed(args.seed)

    def prompt(self) -> list:
        import torch

        return torch.randint(0, self.config.vocab_size, (self.args.prompt_len,), generator=self.gen).tolist()

    def sync(self) -> None:
        import torch

        torch.cuda.synchronize(self.device)

    def decode(self, batch: int, warmup: int, steps: int) -> dict:
        """Decode steps of the continuous-batching engine at this batch size, contexts starting at
        prompt_len: scheduler, step function, sampling on the GPU, tokens to the host."""
        import torch

        from mini_llm_runtime_amd.engine import ContinuousBatchEngine, PageAdmission, Scheduler

        args = self.args
        admission = PageAdmission(self.cache, max_step_tokens=args.prompt_len)
        scheduler = Scheduler(
            max_running_requests=batch,
            max_batch_tokens=max(args.prompt_len, batch),
            admit=admission.admit,
        )
        engine = ContinuousBatchEngine(
            scheduler=scheduler, runner=self.runner, admission=admission, sampler=self.sampler
        )
        for i in range(batch):
            engine.submit(f"b{batch}-{i}", self.prompt(), max_new_tokens=warmup + steps + batch + 8)
        while True:  # prompts, until a step is nothing but one token for every request
            result = engine.step()
            if len(result.plan.decode_ids) == batch:
                break
        for _ in range(warmup):
            engine.step()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        samples = []
        self.sync()
        begin.record()
        t0 = last = time.perf_counter()
        for _ in range(steps):
            result = engine.step()
            now = time.perf_counter()
            samples.append((now - last) * 1e3)
            last = now
        end.record()
        self.sync()
        elapsed = time.perf_counter() - t0
        assert len(result.plan.decode_ids) == batch and len(result.report.emitted) == batch
        engine.run_until_done()
        return {
            "ms": elapsed * 1e3 / steps,
            "ms_device": begin.elapsed_time(end) / steps,
            "samples": samples,
        }

    def kv_bytes_per_token(self) -> int:
        return sum(
            len(g.sites) * g.spec.bytes_per_token(g.key.element_size()) for g in self.cache.groups
        )

    def decode_bytes(self, batch: int, mean_context: float) -> tuple:
        """Bytes a decode step has to read: every weight it uses once, and the live requests' cache."""
        model, config = self.model, self.config
        weight_bytes = model.weight_bytes()
        if not config.tie_word_embeddings:  # an untied input table is only gathered from
            weight_bytes -= model.embed_weight.numel() * model.embed_weight.element_size()
        return weight_bytes, weight_bytes + batch * mean_context * self.kv_bytes_per_token()

    def roofline(self, batch: int, ms: float, warmup: int, steps: int) -> dict:
        _, step_bytes = self.decode_bytes(batch, self.args.prompt_len + warmup + steps / 2)
        achieved = step_bytes / (ms * 1e-3)
        return {
            "bound": "hbm",
            "achieved": round(achieved / 1e9, 1),
            "peak": HBM_BYTES_PER_S / 1e9,
            "unit": "GB/s",
            "frac": round(achieved / HBM_BYTES_PER_S, 4),
        }

    def prefill(self, repeats: int = 5) -> dict:
        """One prompt of prompt_len tokens through the step function, its last logits sampled."""
        import torch

        from mini_llm_runtime_amd.engine.runner import StepEntry
        from mini_llm_runtime_amd.sampling.sampler import GREEDY

        config, tokens = self.config, self.args.prompt_len
        host, dev = [], []
        for i in range(repeats + 1):  # the first run is the warm-up
            rid = f"p{i}"
            self.cache.create_request(rid)
            entry = [StepEntry.of(rid, self.prompt(), (tokens - 1,))]
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            self.sync()
            begin.record()
            t0 = time.perf_counter()
            out = self.runner.step(entry, borrow_logits=True)
            self.sampler.sample(out.logits, [GREEDY], [0]).cpu()
            end.record()
            self.sync()
            host.append((time.perf_counter() - t0) * 1e3)
            dev.append(begin.elapsed_time(end))
            self.cache.release_request(rid)
        host, dev = host[1:], dev[1:]
        ms = sorted(host)[len(host) // 2]
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
        return {
            "value": round(tokens * 1e3 / ms, 1),
            "tokens": tokens,
            "ms": round(ms, 3),
            "frac": round(flops / (ms * 1e-3) / PEAK_FLOPS[self.short], 4),
            "ms_device": round(sorted(dev)[len(dev) // 2], 3),
            "samples_ms": [round(x, 3) for x in host],
        }

    def peak_memory(self) -> dict:
        """Device memory in GiB: the most this process's tensors held at one time since the shape was
        set up (weights, page pool, recorded steps and their buffers; the reference records the same
        counter, src/mini_llm_runtime/timing.py:141-160), the most the allocator had reserved for
        them, and what the driver counts as in use on the device right now."""
        import torch

        free, total = torch.cuda.mem_get_info(self.device)
        gib = float(2**30)
        return {
            "allocated": round(torch.cuda.max_memory_allocated(self.device) / gib, 2),
            "reserved": round(torch.cuda.max_memory_reserved(self.device) / gib, 2),
            "device_in_use": round((total - free) / gib, 2),
        }

    def collect(self) -> None:
        import gc

        import torch

        gc.collect()
        torch.cuda.empty_cache()

    def close(self) -> None:
        for name in ("runner", "cache", "model", "sampler"):
            setattr(self, name, None)
        self.collect()


def large_point(args, name: str, layers, batches=(8,), workload: str = "") -> dict:
    """Decode at the given batch sizes and the prefill for a shape, `layers` of its layers (None: all of
    them), peak device memory, and with `workload` the burst or the chunked workload as a compact
    sub-object."""
    import torch

    bench = Bench(args, name, layers, list(batches))
    try:
        torch.cuda.reset_peak_memory_stats(bench.device)
        warmup, steps = max(2, args.warmup // 2), max(8, args.steps // 2)
        point = {"layers": bench.config.num_hidden_layers, "layers_full_model": bench.full_layers}
        for b in batches:
            run = bench.decode(b, warmup, steps)
            point[f"decode_b{b}"] = round(b * 1e3 / run["ms"], 1)
            point[f"decode_b{b}_ms"] = round(run["ms"], 4)
            if b == 8:
                point["decode_b8_ms_device"] = round(run["ms_device"], 4)
            point[f"decode_b{b}_hbm_frac"] = bench.roofline(b, run["ms"], warmup, steps)["frac"]
        if not args.no_prefill:
            pre = bench.prefill(repeats=3)
            point.update(prefill=pre["value"], prefill_ms=pre["ms"], prefill_frac=pre["frac"])
        point["peak_memory_gb"] = bench.peak_memory()
        if workload:
            bench.runner = bench.cache = None  # the workloads size a cache of their own
            bench.collect()
            line = (burst if workload == "burst" else chunked)(
                args, bench.config, bench.full_layers, bench.model, bench.ops, bench.device
            )
            if workload == "burst":
                point["burst"] = {
                    "generated_tokens_per_s": line["value"],
                    "total_tokens_per_s": line["total_tokens_per_s"],
                    "median_ttft_ms": line["median_ttft_ms"],
                    "median_tpot_ms": line["median_tpot_ms"],
                    "seconds": line["seconds"],
                    "requests": line["config"]["requests"],
                    "max_batch_tokens": line["config"]["max_batch_tokens"],
                }
            else:
                point["chunked"] = {
                    "mixed_step_ms": line["value"],
                    "decoders_tpot_ms_beside_the_prompt": line["decoders_tpot_ms_beside_the_prompt"],
                    "decoders_tpot_ms_alone": line["decoders_tpot_ms_alone"],
                    "prompt_tokens_per_s": line["prompt_tokens_per_s"],
                    "decoders": line["config"]["decoders"],
                    "prompt_len": line["config"]["prompt_len"],
                    "portion": line["config"]["portion"],
                }
        return point
    finally:
        bench.close()


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported", flush=True)
        return 2

    sys.path.insert(0, str(Path(__file__).resolve().parent))
    import mini_llm_runtime_amd  # noqa: F401

    batches = [args.batch] + [int(b) for b in args.points.split(",") if b.strip()]
    bench = Bench(args, args.config, args.layers, batches)
    config = bench.config

    if args.workload in ("library", "reference"):
        line = (library_yardstick if args.workload == "library" else reference_measurements)(args, bench)
        bench.close()
        line["env"] = environment()
        print(json.dumps(line), flush=True)
        return 0
    if args.workload != "decode":
        work = burst if args.workload == "burst" else chunked
        bench.runner = bench.cache = None  # these workloads size a cache of their own
        line = work(args, config, bench.full_layers, bench.model, bench.ops, bench.device)
        line["env"] = environment()
        print(json.dumps(line), flush=True)
        return 0

    default_run = not args.no_large and args.config == "qwen2.5-0.5b" and args.layers is None and args.dtype == "bfloat16"
    main_run = bench.decode(args.batch, args.warmup, args.steps)
    ms_main = main_run["ms"]
    points = {}
    for b in batches[1:]:
        run = bench.decode(b, max(2, args.warmup // 2), max(8, args.steps // 2))
        points[f"decode_b{b}"] = round(b * 1e3 / run["ms"], 1)
    weight_bytes, _ = bench.decode_bytes(args.batch, 0)
    roofline = bench.roofline(args.batch, ms_main, args.warmup, args.steps)
    prefill = None if args.no_prefill else bench.prefill()
    kv_per_token = bench.kv_bytes_per_token()
    full_layers = bench.full_layers
    peak_memory = bench.peak_memory()
    points_reference = None
    if default_run:
        # the reference's own published measurements at their parameters, compact (`--workload reference` has all)
        ours = reference_measurements(args, bench)
        theirs = ours["published"]
        points_reference = {
            "burst_of_8_continuous_tokens_per_s": ours["burst_of_8"]["continuous"]["tokens_per_s"],
            "burst_of_8_static_tokens_per_s": ours["burst_of_8"]["static"]["tokens_per_s"],
            "burst_of_8_continuous_median_ttft_ms": ours["burst_of_8"]["continuous"]["median_ttft_ms"],
            "late_request_ttft_ms_28_and_29_pages": [ours["late_request_under_page_pressure"][k]["ttft_ms"] for k in ("28_blocks", "29_blocks")],
            "prefill_4x512_ms": ours["prefill_4x512_ms"],
            "decode_attention_us": ours["decode_attention_us"],
            "published_rtx3060_fp16": {
                "burst_of_8_continuous_tokens_per_s": theirs["continuous"]["tokens_per_s"],
                "burst_of_8_static_tokens_per_s": theirs["static"]["tokens_per_s"],
                "burst_of_8_continuous_median_ttft_ms": theirs["continuous"]["median_ttft_ms"],
                "late_request_ttft_ms_28_and_29_pages": [theirs["late_request_ttft_ms"]["28_blocks"], theirs["late_request_ttft_ms"]["29_blocks"]],
                "prefill_4x512_ms": theirs["prefill_4x512_ms"],
                "decode_attention_us": theirs["decode_attention_us"],
            },
        }
    bench.close()

    line = {
        "metric": "decode tokens/s",
        "value": round(args.batch * 1e3 / ms_main, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_main, 4),
        "ms_per_step_device": round(main_run["ms_device"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": bench.short,
        "data": "synthetic (random weights made on the device, uniform random token ids)",
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
        "step_samples": summary(main_run["samples"], args.samples),
        "peak_memory_gb": peak_memory,
    }
    if args.tuning:
        line["tuning"] = args.tuning
    if default_run:
        line["points_reference"] = points_reference
        # the other configurations' measurements: decode at batch 1, 8 and 64 and the prefill for the 7B
        # shape and the whole 32B shape (64 layers, 65 GB of weights), the burst of 64 requests on the
        # 7B shape, the 8,192-token prompt in portions beside 32 decoding requests on the 32B shape
        line["points_7b"] = large_point(args, "qwen2.5-7b", None, (1, 8, 64), "burst")
        line["points_32b"] = large_point(args, "qwen2.5-32b", args.layers_32b, (1, 8, 64), "chunked")
        if args.prompt_len == PROMPT_LEN:
            line["points_ctx16k"] = long_context_points(args)
    line["env"] = environment()
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
