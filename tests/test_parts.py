"""Each part a layer is put together from, alone, against the plain function of the same
formula: norm, position encoding, feed-forward, attention mixer (over the paged cache, a
prefix then a portion then single tokens), and the pre-norm block.  On the CPU with the
torch stand-in for the kernels, on the GPU with the HIP kernels."""

from __future__ import annotations

import numpy as np
import pytest
import torch

import plain_qwen2 as plain
from kernel_doubles import TorchOps
from mini_llm_runtime_amd.cache import CacheManager
from mini_llm_runtime_amd.parts import KVView, PartSpec, StepContext, build_part
from mini_llm_runtime_amd.parts.block import PreNormBlock

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


def _tol(dtype):
    return dict(atol=3e-5, rtol=3e-5) if dtype == torch.float32 else dict(atol=3e-2, rtol=3e-2)


def _rand(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale


def _context(ops, cache, entries, dtype, mixer=None):
    """A StepContext for a step of `entries` [(request, new tokens)], as the step function makes it:
    the mixer's own plan for the batch, uploaded and handed out under the plan's key."""
    from types import SimpleNamespace

    from mini_llm_runtime_amd.parts.context import PlanInput

    lay = cache.begin_step(entries)
    dev = ops.device

    def t(a):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    ctx = StepContext(
        ops=ops, dtype=dtype, device=dev, num_tokens=lay.num_tokens, num_entries=lay.num_entries,
        token_ids=t(np.zeros(lay.num_tokens, dtype=np.int32)), positions=t(lay.positions), token_entry=t(lay.token_entry),
        cu_q=t(lay.cu_q), q_starts=t(lay.q_starts), context_lens=t(lay.context_lens),
        max_q_len=int(lay.q_lens.max()), max_context_len=int(lay.context_lens.max()), host=lay,
    )
    plan = mixer.plan(ops, PlanInput(lay.q_lens, lay.q_starts, int(lay.context_lens.max()))) if mixer is not None else None
    if plan is not None:
        ctx.plans[plan.key] = SimpleNamespace(**plan.sizes, **{n: t(a) for n, a in plan.arrays.items()})
    key, value, g = cache.site_pools(0)
    ctx.kv_views[0] = KVView(key, value, t(lay.block_tables[g]), t(lay.slot_mappings[g]), cache.block_size,
                            cache.groups[g].spec.window, True)
    return ctx


@pytest.mark.parametrize("backend,dtype", CASES)
def test_rms_norm_part(backend, dtype):
    ops = _ops(backend, dtype)
    norm = build_part("norm", PartSpec("rms_norm", {"size": 96, "eps": 1e-5}))
    assert norm.param_specs()["weight"].shape == (96,) and norm.param_specs()["weight"].keep_stored_precision
    w = (1 + _rand((96,), 1, 0.1)).to(dtype)
    norm.bind({"weight": w.to(ops.device)}, dtype=dtype, device=ops.device)
    x = _rand((7, 96), 2, 2.0)
    delta = _rand((7, 96), 3).to(dtype)
    ctx = StepContext(ops=ops, dtype=dtype, device=ops.device, num_tokens=7, num_entries=1, token_ids=None, positions=None,
                      token_entry=None, cu_q=None, q_starts=None, context_lens=None, max_q_len=7, max_context_len=7, host=None)
    xd = x.to(ops.device).clone()
    got = norm.forward(ctx, xd, delta.to(ops.device)).cpu()
    summed = x.double() + delta.double()
    torch.testing.assert_close(got.double(), plain.rms_norm(summed, w.double(), 1e-5), **_tol(dtype))
    torch.testing.assert_close(xd.cpu().double(), summed, atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("backend,dtype", CASES[:2])
def test_rotary_part_tables(backend, dtype):
    ops = _ops(backend, dtype)
    rot = build_part("position", PartSpec("rotary", {"head_dim": 32, "theta": 1e6}))
    rot.bind({}, dtype=dtype, device=ops.device)
    pos = torch.tensor([0, 1, 5, 999, 4096], dtype=torch.int32).to(ops.device)
    ctx = StepContext(ops=ops, dtype=dtype, device=ops.device, num_tokens=5, num_entries=1, token_ids=None, positions=pos,
                      token_entry=None, cu_q=None, q_starts=None, context_lens=None, max_q_len=5, max_context_len=5, host=None)
    cos, sin, r = rot.rotation(ctx)
    assert r == 32 and rot.rotation(ctx)[0] is cos  # computed once per step
    ang = plain.rope_angles(pos.cpu(), 32, 1e6)[:, :16]
    torch.testing.assert_close(cos.cpu().double(), ang.cos(), atol=1e-7, rtol=0)
    torch.testing.assert_close(sin.cpu().double(), ang.sin(), atol=1e-7, rtol=0)
    with pytest.raises(ValueError):
        build_part("position", PartSpec("rotary", {"head_dim": 32, "theta": 1e6, "rotary_dim": 34}))


@pytest.mark.parametrize("backend,dtype", CASES)
def test_swiglu_part(backend, dtype):
    ops = _ops(backend, dtype)
    hidden, inter = 96, 352
    ffn = build_part("feed_forward", PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": inter}))
    assert ffn.param_specs()["gate_up_weight"].shape == (2 * inter, hidden)
    w = {"m.gate_proj.weight": _rand((inter, hidden), 4, 0.1).to(dtype), "m.up_proj.weight": _rand((inter, hidden), 5, 0.1).to(dtype),
         "m.down_proj.weight": _rand((hidden, inter), 6, 0.1).to(dtype)}
    woven = torch.empty(2 * inter, hidden, dtype=dtype)
    idx = torch.arange(inter)
    woven[(idx // 2) * 4 + idx % 2] = w["m.gate_proj.weight"]
    woven[(idx // 2) * 4 + 2 + idx % 2] = w["m.up_proj.weight"]
    ffn.bind({"gate_up_weight": woven.to(ops.device), "down_weight": w["m.down_proj.weight"].to(ops.device)}, dtype=dtype, device=ops.device)
    h = _rand((9, hidden), 7).to(dtype)
    ctx = StepContext(ops=ops, dtype=dtype, device=ops.device, num_tokens=9, num_entries=1, token_ids=None, positions=None,
                      token_entry=None, cu_q=None, q_starts=None, context_lens=None, max_q_len=9, max_context_len=9, host=None)
    got = ffn.forward(ctx, h.to(ops.device))
    got = ops.settle(got) if hasattr(ops, "settle") else got  # a part's output may be a product that has not run
    got = got.double().sum(0) if got.dim() == 3 else got.double()
    ref = plain.swiglu(h.double(), {k: v.double() for k, v in w.items()}, "m.")
    torch.testing.assert_close(got.cpu(), ref, **_tol(dtype))


def _attention_part(ops, dtype, heads, kv_heads, head_dim, hidden, theta, seed):
    att = build_part("mixer", PartSpec("gqa_attention", {
        "hidden_size": hidden, "num_heads": heads, "num_kv_heads": kv_heads, "head_dim": head_dim,
        "position": PartSpec("rotary", {"head_dim": head_dim, "theta": theta}),
    }))
    p = "a."
    w = {p + "q_proj.weight": _rand((heads * head_dim, hidden), seed, 0.15), p + "q_proj.bias": _rand((heads * head_dim,), seed + 1, 0.1),
         p + "k_proj.weight": _rand((kv_heads * head_dim, hidden), seed + 2, 0.15), p + "k_proj.bias": _rand((kv_heads * head_dim,), seed + 3, 0.1),
         p + "v_proj.weight": _rand((kv_heads * head_dim, hidden), seed + 4, 0.15), p + "v_proj.bias": _rand((kv_heads * head_dim,), seed + 5, 0.1),
         p + "o_proj.weight": _rand((hidden, heads * head_dim), seed + 6, 0.15)}
    w = {k: v.to(dtype) for k, v in w.items()}
    dev = ops.device
    att.bind({
        "qkv_weight": torch.cat([w[p + "q_proj.weight"], w[p + "k_proj.weight"], w[p + "v_proj.weight"]]).to(dev),
        "qkv_bias_vec": torch.cat([w[p + "q_proj.bias"], w[p + "k_proj.bias"], w[p + "v_proj.bias"]]).to(dev),
        "o_weight": w[p + "o_proj.weight"].to(dev),
    }, dtype=dtype, device=dev)
    att.position.bind({}, dtype=dtype, device=dev)
    return att, w


@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("heads,kv_heads,head_dim,hidden", [(4, 2, 16, 64), (3, 1, 32, 80), (6, 6, 16, 48)])
def test_attention_part_over_the_cache(backend, dtype, heads, kv_heads, head_dim, hidden):
    ops = _ops(backend, dtype)
    att, w = _attention_part(ops, dtype, heads, kv_heads, head_dim, hidden, 10000.0, 10)
    assert att.cache_spec().num_kv_heads == kv_heads and att.cache_spec().window is None
    cache = CacheManager([att.cache_spec()], block_size=8, num_blocks=12, max_requests=2, dtype=dtype, device=ops.device)
    cache.poison()
    cache.create_request("r")
    n = 41
    h = _rand((n, hidden), 20).to(dtype)
    ref = plain.attention_block(h.double(), torch.arange(n), {k: v.double() for k, v in w.items()}, "a.",
                                num_heads=heads, num_kv_heads=kv_heads, head_dim=head_dim, theta=10000.0)
    at = 0
    for size in (19, 13, 1, 1, 5, 1, 1):  # a prefix, a portion behind it, single tokens
        ctx = _context(ops, cache, [("r", size)], dtype, att)
        out = att.forward(ctx, h[at : at + size].to(ops.device), 0)
        out = ops.settle(out) if hasattr(ops, "settle") else out
        out = out.double().sum(0) if out.dim() == 3 else out.double()
        cache.commit_step()
        torch.testing.assert_close(out.cpu(), ref[at : at + size], **_tol(dtype))
        at += size
    assert at == n


@pytest.mark.parametrize("backend,dtype", CASES)
def test_pre_norm_block(backend, dtype):
    ops = _ops(backend, dtype)
    heads, kv_heads, head_dim, hidden, inter = 4, 2, 16, 64, 128
    att, w = _attention_part(ops, dtype, heads, kv_heads, head_dim, hidden, 1e6, 30)
    ffn = build_part("feed_forward", PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": inter}))
    gate, up, down = (_rand(s, 40 + i, 0.1).to(dtype) for i, s in enumerate([(inter, hidden), (inter, hidden), (hidden, inter)]))
    woven = torch.empty(2 * inter, hidden, dtype=dtype)
    idx = torch.arange(inter)
    woven[(idx // 2) * 4 + idx % 2] = gate
    woven[(idx // 2) * 4 + 2 + idx % 2] = up
    ffn.bind({"gate_up_weight": woven.to(ops.device), "down_weight": down.to(ops.device)}, dtype=dtype, device=ops.device)
    norms = {}
    nw = {}
    for i, name in enumerate(("input", "post_mixer")):
        norms[name] = build_part("norm", PartSpec("rms_norm", {"size": hidden, "eps": 1e-6}))
        nw[name] = (1 + _rand((hidden,), 50 + i, 0.1)).to(dtype)
        norms[name].bind({"weight": nw[name].to(ops.device)}, dtype=dtype, device=ops.device)
    block = PreNormBlock(att, ffn, norms)
    weights = {("model.layers.0.self_attn." + k[2:]): v for k, v in w.items()}
    weights.update({"model.layers.0.input_layernorm.weight": nw["input"], "model.layers.0.post_attention_layernorm.weight": nw["post_mixer"],
                    "model.layers.0.mlp.gate_proj.weight": gate, "model.layers.0.mlp.up_proj.weight": up, "model.layers.0.mlp.down_proj.weight": down})
    cfg = dict(rms_norm_eps=1e-6, num_attention_heads=heads, num_key_value_heads=kv_heads, hidden_size=hidden, head_dim=head_dim, rope_theta=1e6)
    n = 23
    x = _rand((n, hidden), 60)
    ref = plain.decoder_layer(x.double(), torch.arange(n), {k: v.double() for k, v in weights.items()}, 0, cfg)
    cache = CacheManager([att.cache_spec()], block_size=8, num_blocks=6, max_requests=1, dtype=dtype, device=ops.device)
    cache.create_request("r")
    ctx = _context(ops, cache, [("r", n)], dtype, att)
    xd = x.to(ops.device).clone()
    stream, delta = block.forward(ctx, xd, None, 0)
    assert stream is xd  # the residual stream is updated in place; the last output is handed on un-added
    delta = ops.settle(delta) if hasattr(ops, "settle") else delta  # the block's last product may not have run
    delta = delta.double().sum(0) if delta.dim() == 3 else delta.double()
    torch.testing.assert_close((stream.double() + delta).cpu(), ref, **_tol(dtype))
