"""Ways of cutting the same requests into steps, in the replay tool's step format
(`{"step": i, "entries": [{"id", "tokens", "want"}], "end": [...]}`), and a driver
that feeds them to a ModelRunner.  The logits at a position must not depend on
the way that was chosen.
"""

from __future__ import annotations

import random
from typing import Mapping, Sequence

import torch

from mini_llm_runtime_amd.cache import blocks_for
from mini_llm_runtime_amd.engine.runner import StepEntry

Requests = Mapping[str, Sequence[int]]


def _step(index: int, entries: list[dict], end: list[str]) -> dict:
    return {"step": index, "entries": entries, "end": end}


def whole(requests: Requests) -> list[dict]:
    """Each request alone and whole, logits everywhere."""
    steps = []
    for rid, toks in requests.items():
        steps.append(_step(len(steps), [{"id": rid, "tokens": list(toks), "want": list(range(len(toks)))}], [rid]))
    return steps


def bulk_then_tail(requests: Requests, tail: int = 32) -> list[dict]:
    """Most of a request in one step, then its last `tail` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        toks = list(toks)
        head = max(1, len(toks) - tail)
        steps.append(_step(len(steps), [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], []))
        for i in range(head, len(toks)):
            steps.append(_step(len(steps), [{"id": rid, "tokens": [toks[i]], "want": [0]}], []))
        steps[-1]["end"] = [rid]
    return steps


def portions(requests: Requests, sizes: Sequence[int] = (7, 2, 16, 3, 2, 5, 11, 2, 4)) -> list[dict]:
    """Portions of changing size, down to two tokens, crossing page edges unaligned."""
    steps = []
    for rid, toks in requests.items():
        toks = list(toks)
        at = 0
        i = 0
        while at < len(toks):
            n = min(sizes[i % len(sizes)], len(toks) - at)
            i += 1
            steps.append(_step(len(steps), [{"id": rid, "tokens": toks[at : at + n], "want": list(range(n))}], []))
            at += n
        steps[-1]["end"] = [rid]
    return steps


def mixed(
    requests: Requests,
    *,
    max_live: int = 4,
    seed: int = 0,
    decode_tail: int = 8,
    max_portion: int = 24,
) -> list[dict]:
    """Up to `max_live` requests at a time: portions of some beside single tokens of
    others; a request may sit a step out; finished requests make room for later ones."""
    rng = random.Random(seed)
    pending = [(rid, list(t)) for rid, t in requests.items()]
    live: dict[str, int] = {}
    steps: list[dict] = []
    while pending or live:
        while pending and len(live) < max_live and (not live or rng.random() < 0.7):
            rid, _ = pending.pop(0)
            live[rid] = 0
        entries, end = [], []
        for rid in list(live):
            toks = list(requests[rid])
            fed = live[rid]
            remaining = len(toks) - fed
            if len(live) > 1 and rng.random() < 0.15:
                continue
            if remaining > decode_tail:
                n = min(remaining - decode_tail, rng.randint(2, max_portion))
                if remaining - decode_tail - n == 1:
                    n += 1
            else:
                n = 1
            entries.append({"id": rid, "tokens": toks[fed : fed + n], "want": list(range(n))})
            live[rid] = fed + n
            if live[rid] == len(toks):
                end.append(rid)
        for rid in end:
            del live[rid]
        if entries:
            steps.append(_step(len(steps), entries, end))
    return steps


def pages_needed(steps: Sequence[dict], block_size: int) -> int:
    """Most pages held at the same time while the steps run."""
    fed: dict[str, int] = {}
    most = 0
    for step in steps:
        for e in step["entries"]:
            fed[e["id"]] = fed.get(e["id"], 0) + len(e["tokens"])
        most = max(most, sum(blocks_for(n, block_size) for n in fed.values()))
        for rid in step["end"]:
            del fed[rid]
    return most


def most_live(steps: Sequence[dict]) -> int:
    live: set[str] = set()
    most = 0
    for step in steps:
        live.update(e["id"] for e in step["entries"])
        most = max(most, len(live))
        live.difference_update(step["end"])
    return most


def run_schedule(runner, cache, steps: Sequence[dict]) -> dict[tuple[str, int], torch.Tensor]:
    """Feed the steps to the runner; returns {(request, absolute position): logits row (CPU float32)}."""
    out: dict[tuple[str, int], torch.Tensor] = {}
    fed: dict[str, int] = {}
    for step in steps:
        entries = []
        for e in step["entries"]:
            if not cache.has_request(e["id"]):
                cache.create_request(e["id"])
                fed[e["id"]] = 0
            entries.append(StepEntry.of(e["id"], e["tokens"], e["want"]))
        result = runner.step(entries)
        if result.logits is not None:
            logits = result.logits.float().cpu()
            for i, (rid, w) in enumerate(result.rows):
                out[(rid, fed[rid] + w)] = logits[i]
        for e in step["entries"]:
            fed[e["id"]] += len(e["tokens"])
        for rid in step["end"]:
            cache.release_request(rid)
            del fed[rid]
    return out
