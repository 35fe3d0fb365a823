"""Generality of the parts: toy parts that exist only in this file are registered,
built into a model by config.json, given random weights, loaded and stepped,
without a change to the framework's files.

* a mixer with state of its own (a causal running mean kept in a per-request
  state slot), in layers that alternate with attention layers;
* an execution order that names a layer twice (two sites, two caches) and lets a
  site read another site's cache;
* attention layers with a window beside layers without (two page pools);
* another position encoding (a learned-free additive ramp applied to q and k);
* a feed-forward with routing (a router, the two best of four experts per token).

None of them is a model of anybody's; they only show that the interfaces hold.
Each is compared with a plain computation written out in this file, whole and in
portions.
"""

from __future__ import annotations

import json
from dataclasses import dataclass, fields
from typing import Any, ClassVar, Mapping

import numpy as np
import pytest
import torch

import mini_llm_runtime_amd as mlr
import plain_qwen2 as plain
from helpers import random_tokens
from kernel_doubles import TorchOps
from mini_llm_runtime_amd.cache import PagedKVSpec, SlotStateSpec
from mini_llm_runtime_amd.config.model_config import ModelConfig
from mini_llm_runtime_amd.engine import ModelRunner, StepEntry
from mini_llm_runtime_amd.models import register_architecture, unregister_architecture
from mini_llm_runtime_amd.parts.context import MixerPlan, PlanInput
from mini_llm_runtime_amd.parts import (
    FeedForward,
    LayerSpec,
    Mixer,
    ModelSpec,
    OrderEntry,
    ParamSpec,
    PartSpec,
    PositionEncoding,
    WeightRule,
    register_part,
    unregister_part,
)
from mini_llm_runtime_amd.weights import SafetensorsFile

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


# ---- toy parts -------------------------------------------------------------------------------------
class RunningMeanMixer(Mixer):
    """out_t = W_out * mean_{i <= t}(W_in h_i): state = the running sum, one vector per request.

    Everything that depends on the step's data happens on the device (sums over the batch's
    tokens, the entries' first tokens from `cu_q`, the state rows from the uploaded metadata),
    so the part says `replayable`: its steps are recorded and replayed like attention's.  It
    also brings a launch plan of its own kind, the index of every entry's last token, which
    the step function uploads without knowing what it is for."""

    replayable = True
    PLAN = "toy_running_mean"

    def __init__(self, hidden_size: int) -> None:
        self.hidden_size = hidden_size
        self.in_weight = None
        self.out_weight = None

    def param_specs(self):
        h = self.hidden_size
        return {"in_weight": ParamSpec((h, h)), "out_weight": ParamSpec((h, h))}

    def cache_spec(self):
        return SlotStateSpec((self.hidden_size,), "float32")

    def plan(self, ops, shape: PlanInput):
        last = np.cumsum(shape.q_lens, dtype=np.int64) - 1
        return MixerPlan(self.PLAN, {"last_token": last.astype(np.int32)}, {"entries": len(shape.q_lens)})

    def forward(self, ctx, h, site):
        ops = ctx.ops
        u = ops.linear(h, self.in_weight, None).double()
        state = ctx.state(site)
        plan = ctx.plan(self.PLAN)
        assert plan.entries == ctx.num_entries and plan.last_token.shape == (ctx.num_entries,)
        sums = torch.cumsum(u, dim=0)  # over the whole batch; each entry subtracts what came before it
        first = ctx.cu_q[:-1].long()
        before = torch.where((first > 0)[:, None], sums[(first - 1).clamp(min=0)], torch.zeros_like(sums[:1]))
        carried = state.tensor[state.read_rows.long()].double() * (ctx.q_starts > 0)[:, None]
        entry = ctx.token_entry.long()
        running = sums - before[entry] + carried[entry]
        out = running / (ctx.positions + 1).double()[:, None]
        state.tensor[state.write_rows.long()] = running[plan.last_token.long()].float()
        return ops.linear(out.to(ctx.dtype), self.out_weight, None)


class RampPosition(PositionEncoding):
    """q and k get `slope * position` added to their first dim: not a rotation, so the
    attention part has to call `apply` and store k without the fused rotation."""

    replayable = True  # nothing here looks at the step's data on the host

    def __init__(self, head_dim: int, slope: float) -> None:
        self.head_dim = head_dim
        self.slope = slope

    def apply(self, ctx, q, k):
        ramp = (ctx.positions.float() * self.slope)[:, None]
        q[:, :, 0] = (q[:, :, 0].float() + ramp).to(q.dtype)
        k[:, :, 0] = (k[:, :, 0].float() + ramp).to(k.dtype)


class RoutedFeedForward(FeedForward):
    """Each token goes to its `top` best of `experts` small two-matrix networks, by a router
    whose logits and softmax are 32-bit; the experts' outputs are added with the renormalised
    router weights.  Which rows an expert gets is decided on the host from the step's data, so
    the part does not say `replayable`."""

    def __init__(self, hidden_size: int, intermediate_size: int, experts: int, top: int, router_scale: float) -> None:
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.experts, self.top, self.router_scale = experts, top, router_scale
        self.router_weight = self.up_weight = self.down_weight = None

    def param_specs(self):
        h, i, e = self.hidden_size, self.intermediate_size, self.experts
        return {"router_weight": ParamSpec((e, h)), "up_weight": ParamSpec((e * i, h)), "down_weight": ParamSpec((e * h, i))}

    def forward(self, ctx, h):
        ops = ctx.ops
        i, width = self.intermediate_size, self.hidden_size
        logits = ops.linear(h, self.router_weight, None, out_dtype=torch.float32) * self.router_scale
        weights, chosen = torch.softmax(logits, dim=-1).topk(self.top, dim=-1)
        weights = weights / weights.sum(dim=-1, keepdim=True)
        out = torch.zeros(h.shape[0], width, dtype=torch.float32, device=h.device)
        for e in range(self.experts):
            rows, slot = (chosen == e).nonzero(as_tuple=True)
            if rows.numel() == 0:
                continue
            inner = ops.linear(h.index_select(0, rows).contiguous(), self.up_weight[e * i : (e + 1) * i], None)
            inner = torch.nn.functional.silu(inner.float()).to(ctx.dtype)
            y = ops.linear(inner, self.down_weight[e * width : (e + 1) * width], None, out_dtype=torch.float32)
            out.index_add_(0, rows, y * weights[rows, slot][:, None])
        return out.to(ctx.dtype)


@dataclass(frozen=True)
class ToyConfig(ModelConfig):
    architecture: ClassVar[str] = "ToyForCausalLM"
    model_type: ClassVar[str] = "toy"
    vocab_size: int = 0
    hidden_size: int = 0
    intermediate_size: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    max_position_embeddings: int = 0
    rms_norm_eps: float = 1e-6
    layer_kinds: tuple = ()  # per layer: "mean", "attention", "window", "ramp"
    order: tuple = ()  # execution sites: (layer, reads_cache_of or -1)
    window: int = 0
    rope_theta: float = 10000.0
    ramp_slope: float = 0.01
    ffn_kinds: tuple = ()  # per layer "swiglu" or "routed"; empty: all "swiglu"
    num_experts: int = 0
    experts_per_token: int = 0
    router_scale: float = 1.0

    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "ToyConfig":
        names = [f.name for f in fields(cls)]
        kw = {n: data[n] for n in names if n in data}
        kw["layer_kinds"] = tuple(kw["layer_kinds"])
        kw["ffn_kinds"] = tuple(kw.get("ffn_kinds", ()))
        kw["order"] = tuple(tuple(o) for o in kw["order"])
        return cls(**kw)

    def to_dict(self):
        d = super().to_dict()
        d["layer_kinds"] = list(self.layer_kinds)
        d["ffn_kinds"] = list(self.ffn_kinds)
        d["order"] = [list(o) for o in self.order]
        return d


def toy_spec(c: ToyConfig) -> ModelSpec:
    norm = PartSpec("rms_norm", {"size": c.hidden_size, "eps": c.rms_norm_eps})
    ffn = PartSpec("swiglu", {"hidden_size": c.hidden_size, "intermediate_size": c.intermediate_size})
    q_rows, kv_rows = c.num_attention_heads * c.head_dim, c.num_key_value_heads * c.head_dim
    layers, rules = [], [WeightRule("embed.weight", "embed.weight"), WeightRule("norm.weight", "final_norm.weight")]
    for i, kind in enumerate(c.layer_kinds):
        p = f"layers.{i}."
        if kind == "mean":
            mixer = PartSpec("toy_running_mean", {"hidden_size": c.hidden_size})
            rules += [WeightRule(p + "mean.in", p + "mixer.in_weight"), WeightRule(p + "mean.out", p + "mixer.out_weight")]
        else:
            position = (
                PartSpec("toy_ramp", {"head_dim": c.head_dim, "slope": c.ramp_slope})
                if kind == "ramp"
                else PartSpec("rotary", {"head_dim": c.head_dim, "theta": c.rope_theta})
            )
            mixer = PartSpec(
                "gqa_attention",
                {
                    "hidden_size": c.hidden_size,
                    "num_heads": c.num_attention_heads,
                    "num_kv_heads": c.num_key_value_heads,
                    "head_dim": c.head_dim,
                    "qkv_bias": False,
                    "position": position,
                    "window": c.window if kind == "window" else None,
                },
            )
            rules += [
                WeightRule(p + "attn.q", p + "mixer.qkv_weight", 0, q_rows),
                WeightRule(p + "attn.k", p + "mixer.qkv_weight", q_rows, kv_rows),
                WeightRule(p + "attn.v", p + "mixer.qkv_weight", q_rows + kv_rows, kv_rows),
                WeightRule(p + "attn.o", p + "mixer.o_weight"),
            ]
        rules += [WeightRule(p + "norm1", p + "norm_input.weight"), WeightRule(p + "norm2", p + "norm_post_mixer.weight")]
        layer_ffn = ffn
        if c.ffn_kinds and c.ffn_kinds[i] == "routed":
            layer_ffn = PartSpec(
                "toy_routed",
                {"hidden_size": c.hidden_size, "intermediate_size": c.intermediate_size, "experts": c.num_experts,
                 "top": c.experts_per_token, "router_scale": c.router_scale},
            )
            rules += [
                WeightRule(p + "ffn.router", p + "feed_forward.router_weight"),
                WeightRule(p + "ffn.experts.up", p + "feed_forward.up_weight"),
                WeightRule(p + "ffn.experts.down", p + "feed_forward.down_weight"),
            ]
        else:
            rules += [
                WeightRule(p + "ffn.gate", p + "feed_forward.gate_up_weight", 0, c.intermediate_size, block=2, period=4),
                WeightRule(p + "ffn.up", p + "feed_forward.gate_up_weight", 2, c.intermediate_size, block=2, period=4),
                WeightRule(p + "ffn.down", p + "feed_forward.down_weight"),
            ]
        layers.append(LayerSpec("pre_norm", mixer, layer_ffn, {"input": norm, "post_mixer": norm}))
    return ModelSpec(
        architecture=c.architecture,
        vocab_size=c.vocab_size,
        hidden_size=c.hidden_size,
        max_position_embeddings=c.max_position_embeddings,
        layers=tuple(layers),
        order=tuple(OrderEntry(l, None if src < 0 else src) for l, src in c.order),
        final_norm=norm,
        tie_word_embeddings=True,
        weight_rules=tuple(rules),
        init_std=0.05,
    )


@pytest.fixture()
def toy_registered():
    register_part("mixer", "toy_running_mean", RunningMeanMixer, replace=True)
    register_part("position", "toy_ramp", RampPosition, replace=True)
    register_part("feed_forward", "toy_routed", RoutedFeedForward, replace=True)
    register_architecture("ToyForCausalLM", ToyConfig, toy_spec, replace=True)
    yield
    unregister_architecture("ToyForCausalLM")
    unregister_part("mixer", "toy_running_mean")
    unregister_part("position", "toy_ramp")
    unregister_part("feed_forward", "toy_routed")


# ---- the plain computation of the same toy model ------------------------------------------------------
def toy_plain(tokens, w, c: ToyConfig, gaps=None):
    """Logits of the whole sequence.  `gaps` collects, per routed layer, each token's router
    logit gap between its last chosen and its first rejected expert, relative to its largest logit."""
    x = w["embed.weight"].double()[torch.tensor(tokens)]
    n = len(tokens)
    pos = torch.arange(n)
    cached_kv = {}
    for site, (layer, src) in enumerate(c.order):
        p = f"layers.{layer}."
        kind = c.layer_kinds[layer]
        h = plain.rms_norm(x, w[p + "norm1"].double(), c.rms_norm_eps)
        if kind == "mean":
            u = h @ w[p + "mean.in"].double().t()
            mean = torch.cumsum(u, 0) / torch.arange(1, n + 1)[:, None]
            mixed = mean @ w[p + "mean.out"].double().t()
        else:
            hq, hkv, d = c.num_attention_heads, c.num_key_value_heads, c.head_dim
            q = (h @ w[p + "attn.q"].double().t()).view(n, hq, d).transpose(0, 1)
            if src < 0:
                k = (h @ w[p + "attn.k"].double().t()).view(n, hkv, d).transpose(0, 1)
                v = (h @ w[p + "attn.v"].double().t()).view(n, hkv, d).transpose(0, 1)
            if kind == "ramp":
                q = q.clone()
                q[:, :, 0] += pos * c.ramp_slope
                if src < 0:
                    k = k.clone()
                    k[:, :, 0] += pos * c.ramp_slope
            else:
                q = plain.apply_rope(q, pos, c.rope_theta)
                if src < 0:
                    k = plain.apply_rope(k, pos, c.rope_theta)
            if src < 0:
                cached_kv[site] = (k, v)
            else:
                k, v = cached_kv[src]  # this site reads the other site's keys and values
            att = plain.causal_attention(q, k, v, window=c.window if kind == "window" else None)
            mixed = att.transpose(0, 1).reshape(n, hq * d) @ w[p + "attn.o"].double().t()
        x = x + mixed
        h = plain.rms_norm(x, w[p + "norm2"].double(), c.rms_norm_eps)
        if c.ffn_kinds and c.ffn_kinds[layer] == "routed":
            i, width = c.intermediate_size, c.hidden_size
            logits = (h @ w[p + "ffn.router"].double().t()) * c.router_scale
            ordered = logits.sort(dim=-1, descending=True).values
            if gaps is not None:
                gaps.append((ordered[:, c.experts_per_token - 1] - ordered[:, c.experts_per_token]) / logits.abs().max(-1).values)
            weights, chosen = torch.softmax(logits, -1).topk(c.experts_per_token, -1)
            weights = weights / weights.sum(-1, keepdim=True)
            y = torch.zeros_like(x)
            for t in range(n):
                for weight, e in zip(weights[t], chosen[t]):
                    up = w[p + "ffn.experts.up"].double()[int(e) * i : (int(e) + 1) * i]
                    down = w[p + "ffn.experts.down"].double()[int(e) * width : (int(e) + 1) * width]
                    y[t] += weight * (down @ torch.nn.functional.silu(up @ h[t]))
            x = x + y
            continue
        g = h @ w[p + "ffn.gate"].double().t()
        x = x + (g * torch.sigmoid(g) * (h @ w[p + "ffn.up"].double().t())) @ w[p + "ffn.down"].double().t()
    x = plain.rms_norm(x, w["norm.weight"].double(), c.rms_norm_eps)
    return x @ w["embed.weight"].double().t()


TOYS = {
    # a mixer with state of its own between attention layers; layer 1 runs twice
    "state": dict(layer_kinds=["attention", "mean", "attention"], order=[[0, -1], [1, -1], [2, -1], [1, -1]], window=0),
    # window layers beside full layers (two page pools), a site that reads another site's cache, another position encoding
    "window": dict(layer_kinds=["window", "attention", "ramp"], order=[[0, -1], [1, -1], [2, -1], [1, 1], [0, -1]], window=11),
}


def _toy_config(name):
    base = dict(
        architectures=["ToyForCausalLM"], model_type="toy", vocab_size=97, hidden_size=48, intermediate_size=80,
        num_attention_heads=3, num_key_value_heads=1, head_dim=16, max_position_embeddings=256, rms_norm_eps=1e-5,
    )
    base.update(TOYS[name])
    return base


@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("name", list(TOYS))
def test_toy_model_whole_and_in_portions(tmp_path, toy_registered, name, backend, dtype):
    config = mlr.models.config_from_dict(_toy_config(name))
    assert isinstance(config, ToyConfig)
    folder = mlr.write_random_model(config, tmp_path / name, seed=7)
    assert json.loads((folder / "config.json").read_text())["architectures"] == ["ToyForCausalLM"]
    with SafetensorsFile(folder / "model.safetensors") as f:
        weights = {n: f.tensor(n) for n in f.entries}
    ops = _ops(backend, dtype)
    cfg, model = mlr.load_model(folder, dtype=dtype, device=ops.device)
    specs = model.site_cache_specs()
    if name == "state":
        assert [type(s).__name__ for s in specs] == ["PagedKVSpec", "SlotStateSpec", "PagedKVSpec", "SlotStateSpec"]
    else:
        assert specs[3] is None and specs[0] == PagedKVSpec(1, 16, 11) and specs[1] == PagedKVSpec(1, 16, None)
    cache = mlr.make_cache(model, block_size=4, num_blocks=24, max_requests=3)
    if name == "window":
        assert len(cache.groups) == 2 and cache.groups[0].sites == (0, 4) and cache.groups[1].sites == (1, 2)
    cache.poison()
    runner = ModelRunner(model, cache, ops)
    requests = {"a": random_tokens(45, 97, 1), "b": random_tokens(23, 97, 2)}
    refs = {rid: toy_plain(toks, weights, config) for rid, toks in requests.items()}

    def check(got, rid, base):
        ref = refs[rid][base : base + got.shape[0]]
        err = (got.double().cpu() - ref).abs().max() / ref.abs().max()
        assert err < (1e-4 if dtype == torch.float32 else 4e-2), (rid, base, float(err))

    # whole
    for rid, toks in requests.items():
        cache.create_request(rid)
        out = runner.step([StepEntry.of(rid, toks, range(len(toks)))])
        check(out.logits, rid, 0)
        cache.release_request(rid)
    # portions, both requests in one batch, single tokens at the end, one aborted step in between
    fed = {rid: 0 for rid in requests}
    for rid in requests:
        cache.create_request(rid)
    sizes = [5, 2, 9, 3, 1, 1, 7, 1, 4, 6, 1, 1, 1, 8, 2]
    i = 0
    while any(fed[r] < len(requests[r]) for r in requests):
        entries = []
        for rid, toks in requests.items():
            n = min(sizes[(i + (rid == "b")) % len(sizes)], len(toks) - fed[rid])
            if n > 0:
                entries.append(StepEntry.of(rid, toks[fed[rid] : fed[rid] + n], range(n)))
        if i == 3:  # a failed step must leave pages and state as they were
            runner.fail_next_step = RuntimeError("injected")
            with pytest.raises(RuntimeError, match="injected"):
                runner.step(entries)
        out = runner.step(entries)
        at = 0
        for e in entries:
            check(out.logits[at : at + len(e.tokens)], e.request_id, fed[e.request_id])
            at += len(e.tokens)
            fed[e.request_id] += len(e.tokens)
        i += 1
        cache.check_invariants()
    if name == "window":  # the window pool gave pages back while the full pool kept them
        a = cache.get_request("a")
        assert a.tables[0][0] == -1 and len(a.live_blocks(0)) < len(a.live_blocks(1))
    for rid in requests:
        cache.release_request(rid)
    assert all(g.allocator.free_count == g.num_blocks for g in cache.groups)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_steps_of_a_model_with_state_are_recorded(tmp_path, toy_registered, dtype):
    """Fixed-size state is no obstacle to recordings: a model with the running-mean mixer decodes
    through replayed graphs (batches of 1, 2 and 3 requests, padded to 1, 2 and 4 entries, the
    padded one on the banks' spare rows) and repeats prompt portions through recorded steps, all
    bit for bit what plain steps give, and the requests' states stay their own."""
    from mini_llm_runtime_amd.kernels.ops import HipOps

    config = mlr.models.config_from_dict(_toy_config("state"))
    folder = mlr.write_random_model(config, tmp_path / "state", seed=8)
    with SafetensorsFile(folder / "model.safetensors") as f:
        weights = {n: f.tensor(n) for n in f.entries}
    requests = {"a": random_tokens(60, 97, 3), "b": random_tokens(49, 97, 4), "c": random_tokens(38, 97, 5)}
    refs = {rid: toy_plain(toks, weights, config) for rid, toks in requests.items()}
    outputs = {}
    for graphs in (False, True):
        ops = HipOps(dtype, "cuda")
        _, model = mlr.load_model(folder, dtype=dtype, device=ops.device)
        assert model.replayable
        cache = mlr.make_cache(model, block_size=4, num_blocks=64, max_requests=3)
        cache.poison()
        runner = ModelRunner(model, cache, ops, use_graphs=graphs)
        got = []
        fed = {}
        for rid, toks in requests.items():  # prompts in portions of 8: the same sizes again and again
            cache.create_request(rid)
            for at in range(0, 24, 8):
                got.append(runner.step([StepEntry.of(rid, toks[at : at + 8], range(8))]).logits)
            fed[rid] = 24
        live = list(requests)
        while live:  # one token each; requests end one after the other: batches of 3, 2, 1
            entries = [StepEntry.of(rid, [requests[rid][fed[rid]]], (0,)) for rid in live]
            out = runner.step(entries).logits
            got.append(out)
            for i, rid in enumerate(live):
                ref = refs[rid][fed[rid]]
                err = (out[i].double().cpu() - ref).abs().max() / ref.abs().max()
                assert err < (1e-4 if dtype == torch.float32 else 4e-2), (rid, fed[rid], float(err))
                fed[rid] += 1
            live = [rid for rid in live if fed[rid] < len(requests[rid])]
        outputs[graphs] = got
        if graphs:
            assert set(runner._graphs) == {(1, 256), (2, 256), (4, 256)}, "single-token steps were not recorded"
            assert len(runner._step_graphs) == 1, "the repeated portions were not recorded"
        for rid in requests:
            cache.release_request(rid)
    for i, (want, have) in enumerate(zip(outputs[False], outputs[True])):
        assert torch.equal(want, have), f"step {i}: a replayed step differs from the plain one"


ROUTED = dict(
    layer_kinds=["attention", "attention", "attention"], ffn_kinds=["swiglu", "routed", "swiglu"],
    order=[[0, -1], [1, -1], [2, -1]], window=0, num_experts=4, experts_per_token=2, router_scale=30.0,
)


@pytest.mark.parametrize("backend,dtype", CASES)
def test_toy_routed_feed_forward(tmp_path, toy_registered, backend, dtype):
    """A feed-forward with a router and experts, defined above, in one of three layers: whole
    prompts, then portions of two requests in one batch with single tokens at the end.  Random
    weights can leave a token on the edge between two experts, where bfloat16 may choose the
    other one; the seed is the first whose routing is clear for every token (32-bit needs none)."""
    base = dict(
        architectures=["ToyForCausalLM"], model_type="toy", vocab_size=97, hidden_size=48, intermediate_size=40,
        num_attention_heads=3, num_key_value_heads=1, head_dim=16, max_position_embeddings=256, rms_norm_eps=1e-5,
    )
    base.update(ROUTED)
    config = mlr.models.config_from_dict(base)
    requests = {"a": random_tokens(23, 97, 11), "b": random_tokens(11, 97, 12)}
    for seed in range(20, 120):
        folder = mlr.write_random_model(config, tmp_path / f"routed{seed}", seed=seed)
        with SafetensorsFile(folder / "model.safetensors") as f:
            weights = {n: f.tensor(n) for n in f.entries}
        gaps: list = []
        refs = {rid: toy_plain(toks, weights, config, gaps) for rid, toks in requests.items()}
        if min(float(g.min()) for g in gaps) > 0.06:
            break
    else:
        pytest.fail("no seed with clear routing")
    assert len(gaps) == 2 and {n for n in weights if "router" in n} == {"layers.1.ffn.router"}
    ops = _ops(backend, dtype)
    cfg, model = mlr.load_model(folder, dtype=dtype, device=ops.device)
    assert not model.replayable  # the routed part plans on the host: its steps are never recorded
    cache = mlr.make_cache(model, block_size=4, num_blocks=24, max_requests=2)
    cache.poison()
    runner = ModelRunner(model, cache, ops)

    def check(got, rid, first):
        ref = refs[rid][first : first + got.shape[0]]
        err = (got.double().cpu() - ref).abs().max() / ref.abs().max()
        assert err < (1e-4 if dtype == torch.float32 else 4e-2), (rid, first, float(err))

    for rid, toks in requests.items():
        cache.create_request(rid)
        check(runner.step([StepEntry.of(rid, toks, range(len(toks)))]).logits, rid, 0)
        cache.release_request(rid)
    fed = {rid: 0 for rid in requests}
    for rid in requests:
        cache.create_request(rid)
    sizes = [6, 1, 3, 9, 1, 1, 2, 5]
    i = 0
    while any(fed[r] < len(requests[r]) for r in requests):
        entries = []
        for rid, toks in requests.items():
            n = min(sizes[(i + 3 * (rid == "b")) % len(sizes)], len(toks) - fed[rid])
            if n > 0:
                entries.append(StepEntry.of(rid, toks[fed[rid] : fed[rid] + n], range(n)))
        out = runner.step(entries)  # the same sizes come again and again: still no recording
        at = 0
        for e in entries:
            check(out.logits[at : at + len(e.tokens)], e.request_id, fed[e.request_id])
            at += len(e.tokens)
            fed[e.request_id] += len(e.tokens)
        i += 1
    assert not getattr(runner, "_step_graphs", {})
    for rid in requests:
        cache.release_request(rid)
    assert all(g.allocator.free_count == g.num_blocks for g in cache.groups)


def test_unknown_part_kind_is_named(toy_registered):
    bad = _toy_config("state")
    config = mlr.models.config_from_dict(bad)
    unregister_part("mixer", "toy_running_mean")
    with pytest.raises(KeyError, match="toy_running_mean.*gqa_attention"):
        mlr.build_model(config)
