"""Other kinds of cache, defined in this file only: nothing under `mini_llm_runtime_amd/` knows them.

* `LatentPagesSpec`: a THIRD kind of site cache beside paged keys/values and fixed-size slots: one
  compressed vector per token in pages of its own geometry ([page, offset, latent], no heads, no
  values), with a view class of its own.  The cache manager gives it a pool, block tables, page reuse
  and the step transaction because the spec attaches itself to the paged store; the step function hands
  the mixer whatever view the spec makes.
* `RowMajorValuesSpec`: paged keys and values in ANOTHER LAYOUT (values [page, kv_head, offset, dim],
  not transposed), by overriding the spec's page shapes.
* a launch plan that is made from the step's `StepLayout` and token ids (request slots, each entry's
  first token), which `PlanInput` carries.

A two-layer toy model uses both; it is compared with a plain computation, whole, in portions and
mixed with other requests on so few pages that they are used again.
"""

from __future__ import annotations

import json
from dataclasses import dataclass, fields
from typing import Any, ClassVar, Mapping, Optional

import numpy as np
import pytest
import torch

import mini_llm_runtime_amd as mlr
import plain_qwen2 as plain
import schedules
from helpers import random_tokens
from kernel_doubles import TorchOps
from mini_llm_runtime_amd.cache import PagedKVSpec, PagedSpec
from mini_llm_runtime_amd.config.model_config import ModelConfig
from mini_llm_runtime_amd.engine import ModelRunner
from mini_llm_runtime_amd.engine.factory import page_bytes
from mini_llm_runtime_amd.models import config_from_dict, register_architecture, unregister_architecture
from mini_llm_runtime_amd.parts import (
    LayerSpec,
    Mixer,
    ModelSpec,
    OrderEntry,
    ParamSpec,
    PartSpec,
    WeightRule,
    register_part,
    unregister_part,
)
from mini_llm_runtime_amd.parts.context import MixerPlan, PlanInput

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


# ---- a third kind of cache: one latent vector per token, in pages of its own shape -------------------------
@dataclass
class LatentView:
    latent: torch.Tensor  # [page, offset, latent]
    block_table: torch.Tensor
    slot_mapping: torch.Tensor
    block_size: int
    writable: bool


@dataclass(frozen=True)
class LatentPagesSpec(PagedSpec):
    latent_dim: int
    window: Optional[int] = None

    def bytes_per_token(self, element_size: int) -> int:
        return self.latent_dim * 4  # kept in 32-bit whatever the engine computes in

    def page_tensors(self, sites, num_blocks, block_size, dtype, device):
        return {"latent": torch.empty((sites, num_blocks, block_size, self.latent_dim), dtype=torch.float32, device=device)}

    def view(self, pages, *, block_table, slot_mapping, block_size, writable, **_):
        return LatentView(pages["latent"], block_table, slot_mapping, block_size, writable)


class LatentMeanMixer(Mixer):
    """c_t = W_c h_t is cached per token; out_t = W_out mean_{i <= t} c_i, read back from the pages.
    Its plan is made from the step's layout and token ids."""

    PLAN = "toy_latent"
    seen_plans: ClassVar[list] = []  # (request slots, first tokens) of every step, for the test

    def __init__(self, hidden_size: int, latent_dim: int) -> None:
        self.hidden_size, self.latent_dim = hidden_size, latent_dim
        self.c_weight = self.out_weight = None

    def param_specs(self):
        return {"c_weight": ParamSpec((self.latent_dim, self.hidden_size)), "out_weight": ParamSpec((self.hidden_size, self.latent_dim))}

    def cache_spec(self):
        return LatentPagesSpec(self.latent_dim)

    def plan(self, ops, shape: PlanInput):
        entries = len(shape.q_lens)
        slots = np.full(entries, -1, dtype=np.int32)
        first = np.full(entries, -1, dtype=np.int32)
        if shape.layout is not None:  # (None: the probe when the runner is built)
            real = shape.layout.num_entries
            slots[:real] = shape.layout.slots
            first[:real] = shape.token_ids[shape.layout.cu_q[:-1]]
        return MixerPlan(self.PLAN, {"request_slots": slots, "first_token": first}, {"entries": entries})

    def forward(self, ctx, h, site):
        ops = ctx.ops
        cache = ctx.cache(site)
        assert isinstance(cache, LatentView) and cache.writable
        plan = ctx.plan(self.PLAN)
        LatentMeanMixer.seen_plans.append((plan.request_slots.cpu().tolist(), plan.first_token.cpu().tolist()))
        c = ops.linear(h, self.c_weight, None, out_dtype=torch.float32)
        flat = cache.latent.view(-1, self.latent_dim)  # [page * block_size + offset, latent]
        flat[cache.slot_mapping.long()] = c
        bs = cache.block_size
        out = torch.empty(h.shape[0], self.latent_dim, dtype=torch.float32, device=h.device)
        table = cache.block_table.long()
        for t in range(h.shape[0]):  # from the pages, whatever was cut where
            entry, pos = int(ctx.token_entry[t]), int(ctx.positions[t])
            idx = torch.arange(pos + 1, device=h.device)
            rows = table[entry, idx // bs] * bs + idx % bs
            out[t] = flat[rows].mean(0)
        return ops.linear(out.to(ctx.dtype), self.out_weight, None)


# ---- keys and values in another page layout ------------------------------------------------------------------
@dataclass(frozen=True)
class RowMajorValuesSpec(PagedKVSpec):
    def value_page_shape(self, block_size: int):
        return (self.num_kv_heads, block_size, self.value_dim)  # a token's value contiguous, like its key


class PlainPagedAttention(Mixer):
    """Causal attention without position encoding, computed with torch from pages whose values are
    not transposed."""

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int) -> None:
        self.hidden_size, self.num_heads, self.head_dim = hidden_size, num_heads, head_dim
        self.qkv_weight = self.o_weight = None

    def param_specs(self):
        width = 3 * self.num_heads * self.head_dim
        return {"qkv_weight": ParamSpec((width, self.hidden_size)), "o_weight": ParamSpec((self.hidden_size, self.num_heads * self.head_dim))}

    def cache_spec(self):
        return RowMajorValuesSpec(self.num_heads, self.head_dim)

    def forward(self, ctx, h, site):
        ops = ctx.ops
        cache = ctx.kv(site)
        heads, d, bs = self.num_heads, self.head_dim, cache.block_size
        assert cache.key.shape[1:] == (heads, bs, d) and cache.value.shape[1:] == (heads, bs, d), "the spec's layout"
        qkv = ops.linear(h, self.qkv_weight, None, out_dtype=torch.float32).view(-1, 3, heads, d)
        slots = cache.slot_mapping.long()
        cache.key[slots // bs, :, slots % bs] = qkv[:, 1].to(cache.key.dtype)
        cache.value[slots // bs, :, slots % bs] = qkv[:, 2].to(cache.value.dtype)
        cache.written()
        cache.reading()
        table = cache.block_table.long()
        out = torch.empty(h.shape[0], heads, d, dtype=torch.float32, device=h.device)
        for t in range(h.shape[0]):
            entry, pos = int(ctx.token_entry[t]), int(ctx.positions[t])
            idx = torch.arange(pos + 1, device=h.device)
            page, off = table[entry, idx // bs], idx % bs
            k = cache.key[page, :, off].float()  # [n, heads, d]
            v = cache.value[page, :, off].float()
            s = torch.einsum("hd,nhd->hn", qkv[t, 0], k) * d**-0.5
            out[t] = torch.einsum("hn,nhd->hd", torch.softmax(s, -1), v)
        return ops.linear(out.view(-1, heads * d).to(ctx.dtype), self.o_weight, None)


# ---- a toy architecture of the two ----------------------------------------------------------------------------
@dataclass(frozen=True)
class KindsConfig(ModelConfig):
    architecture: ClassVar[str] = "ToyKindsForCausalLM"
    model_type: ClassVar[str] = "toy_kinds"
    vocab_size: int = 0
    hidden_size: int = 0
    intermediate_size: int = 0
    latent_dim: int = 0
    num_attention_heads: int = 0
    head_dim: int = 0
    max_position_embeddings: int = 0
    rms_norm_eps: float = 1e-6

    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "KindsConfig":
        return cls(**{f.name: data[f.name] for f in fields(cls) if f.name in data})


def kinds_spec(c: KindsConfig) -> ModelSpec:
    norm = PartSpec("rms_norm", {"size": c.hidden_size, "eps": c.rms_norm_eps})
    ffn = PartSpec("swiglu", {"hidden_size": c.hidden_size, "intermediate_size": c.intermediate_size})
    mixers = [
        PartSpec("toy_latent_mean", {"hidden_size": c.hidden_size, "latent_dim": c.latent_dim}),
        PartSpec("toy_plain_attention", {"hidden_size": c.hidden_size, "num_heads": c.num_attention_heads, "head_dim": c.head_dim}),
    ]
    rules = [WeightRule("embed.weight", "embed.weight"), WeightRule("norm.weight", "final_norm.weight")]
    for i, names in enumerate((("c_weight", "out_weight"), ("qkv_weight", "o_weight"))):
        p = f"layers.{i}."
        rules += [WeightRule(p + n, p + "mixer." + n) for n in names]
        rules += [
            WeightRule(p + "norm1", p + "norm_input.weight"), WeightRule(p + "norm2", p + "norm_post_mixer.weight"),
            WeightRule(p + "ffn.gate", p + "feed_forward.gate_up_weight", 0, c.intermediate_size, block=2, period=4),
            WeightRule(p + "ffn.up", p + "feed_forward.gate_up_weight", 2, c.intermediate_size, block=2, period=4),
            WeightRule(p + "ffn.down", p + "feed_forward.down_weight"),
        ]
    return ModelSpec(
        architecture=c.architecture, vocab_size=c.vocab_size, hidden_size=c.hidden_size,
        max_position_embeddings=c.max_position_embeddings,
        layers=tuple(LayerSpec("pre_norm", m, ffn, {"input": norm, "post_mixer": norm}) for m in mixers),
        order=(OrderEntry(0), OrderEntry(1)), final_norm=norm, tie_word_embeddings=True, weight_rules=tuple(rules), init_std=0.05,
    )


@pytest.fixture()
def kinds_registered():
    register_part("mixer", "toy_latent_mean", LatentMeanMixer, replace=True)
    register_part("mixer", "toy_plain_attention", PlainPagedAttention, replace=True)
    register_architecture(KindsConfig.architecture, KindsConfig, kinds_spec, replace=True)
    LatentMeanMixer.seen_plans.clear()
    yield
    unregister_architecture(KindsConfig.architecture)
    unregister_part("mixer", "toy_latent_mean")
    unregister_part("mixer", "toy_plain_attention")


CONFIG = dict(architectures=["ToyKindsForCausalLM"], model_type="toy_kinds", vocab_size=211, hidden_size=48, intermediate_size=80,
              latent_dim=12, num_attention_heads=3, head_dim=8, max_position_embeddings=256, rms_norm_eps=1e-5)


def kinds_plain(tokens, w, c: KindsConfig):
    x = w["embed.weight"].double()[torch.tensor(tokens)]
    n = len(tokens)
    for i in range(2):
        p = f"layers.{i}."
        h = plain.rms_norm(x, w[p + "norm1"].double(), c.rms_norm_eps)
        if i == 0:
            latent = h @ w[p + "c_weight"].double().t()
            mean = torch.cumsum(latent, 0) / torch.arange(1, n + 1)[:, None]
            mixed = mean @ w[p + "out_weight"].double().t()
        else:
            qkv = (h @ w[p + "qkv_weight"].double().t()).view(n, 3, c.num_attention_heads, c.head_dim)
            q, k, v = (qkv[:, j].transpose(0, 1) for j in range(3))
            att = plain.causal_attention(q, k, v)
            mixed = att.transpose(0, 1).reshape(n, -1) @ w[p + "o_weight"].double().t()
        x = x + mixed
        h = plain.rms_norm(x, w[p + "norm2"].double(), c.rms_norm_eps)
        gate, up = h @ w[p + "ffn.gate"].double().t(), h @ w[p + "ffn.up"].double().t()
        x = x + (torch.nn.functional.silu(gate) * up) @ w[p + "ffn.down"].double().t()
    x = plain.rms_norm(x, w["norm.weight"].double(), c.rms_norm_eps)
    return x @ w["embed.weight"].double().t()


@pytest.mark.parametrize("backend,dtype", CASES)
def test_a_third_cache_kind_and_another_page_layout_need_no_framework_change(tmp_path, kinds_registered, backend, dtype):
    from mini_llm_runtime_amd.weights import SafetensorsFile

    config = config_from_dict(CONFIG)
    folder = mlr.write_random_model(config, tmp_path / "kinds", seed=5, storage_dtype="float32")
    with SafetensorsFile(folder / "model.safetensors") as f:
        weights = {n: f.tensor(n) for n in f.entries}
    ops = _ops(backend, dtype)
    _, model = mlr.load_model(folder, dtype=dtype, device=ops.device)
    requests = {f"r{i}": random_tokens(n, CONFIG["vocab_size"], 40 + i) for i, n in enumerate((5, 19, 33, 26, 41))}
    bs = 4
    for family in (schedules.whole, schedules.portions, lambda r: schedules.mixed(r, seed=2)):
        steps = family(requests)
        pages = schedules.pages_needed(steps, bs)
        cache = mlr.make_cache(model, block_size=bs, num_blocks=pages, max_requests=4)
        # two pools, because the two sites' specs differ; each with the tensors its spec made
        assert len(cache.groups) == 2
        latent, attention = cache.groups
        assert set(latent.tensors) == {"latent"} and latent.tensors["latent"].shape == (1, pages, bs, 12)
        assert latent.tensors["latent"].dtype == torch.float32
        assert attention.value.shape == (1, pages, 3, bs, 8) and attention.key.shape == (1, pages, 3, bs, 8)
        assert page_bytes(model, bs, dtype) == bs * (12 * 4 + 2 * 3 * 8 * torch.empty((), dtype=dtype).element_size())
        cache.poison()
        runner = ModelRunner(model, cache, ops)
        LatentMeanMixer.seen_plans.clear()
        got = schedules.run_schedule(runner, cache, steps)
        cache.check_invariants()
        assert cache.request_ids == () and all(g.allocator.free_count == g.num_blocks for g in cache.groups)
        for rid, toks in requests.items():
            ref = kinds_plain(toks, weights, config)
            for pos in range(len(toks)):
                row = got[(rid, pos)].double()
                if dtype == torch.float32:
                    assert float((row - ref[pos]).abs().max()) < 1e-4, (rid, pos)
                else:
                    assert float((row - ref[pos]).norm() / ref[pos].norm()) < 5e-2, (rid, pos)
        # the plan saw the layout and the token ids of every step
        assert len(LatentMeanMixer.seen_plans) == len(steps)
        for (slots, first), step in zip(LatentMeanMixer.seen_plans, steps):
            assert first[: len(step["entries"])] == [e["tokens"][0] for e in step["entries"]]
            assert len(set(slots[: len(step["entries"])])) == len(step["entries"]) and min(slots[: len(step["entries"])]) >= 0
