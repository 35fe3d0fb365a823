"""What another architecture would need of the framework without a change to its files, shown
with toy parts and toy specs that exist only here: checkpoints that store several parameters
in one tensor (fused, stacked, transposed), what some decoders do around the layers (a scale
on the embedding, an added position embedding, a bias and a soft cap on the logits), caches
whose values are narrower than their keys or absent, and parts that need whole prompts."""

from __future__ import annotations

import dataclasses
import json

import pytest
import torch

import mini_llm_runtime_amd as mlr
import plain_qwen2 as plain
from helpers import StepEntry, TINY, make_model_dir, random_tokens, read_weights
from kernel_doubles import TorchOps
from mini_llm_runtime_amd.cache import CacheManager, PagedKVSpec
from mini_llm_runtime_amd.config import Qwen2Config
from mini_llm_runtime_amd.engine import ContinuousBatchEngine, ModelRunner, PageAdmission, Scheduler
from mini_llm_runtime_amd.engine.factory import page_bytes
from mini_llm_runtime_amd.models.qwen2 import qwen2_spec
from mini_llm_runtime_amd.parts import DecoderModel, ParamSpec, PartSpec, PositionEncoding, WeightRule, register_part, unregister_part
from mini_llm_runtime_amd.parts.attention import GQAAttention
from mini_llm_runtime_amd.weights import WeightsError, load_weights
from mini_llm_runtime_amd.weights.safetensors_io import write_safetensors

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


# ---- one stored tensor, several parameters ---------------------------------------------------------------
def _packed_rules(config: Qwen2Config, spec):
    """The Qwen2 rules rewritten for a checkpoint that stores q, k and v of a layer as one matrix
    `qkv_proj`, gate and up as one matrix `gate_up_proj`, the down matrices of all layers stacked
    in one tensor `model.down_stack` [layers, hidden, intermediate], and o transposed."""
    d = config.head_dim
    q_rows, kv_rows, inter, hidden = config.num_attention_heads * d, config.num_key_value_heads * d, config.intermediate_size, config.hidden_size
    width = q_rows + 2 * kv_rows
    rules = []
    for rule in spec.weight_rules:
        if any(k in rule.name for k in ("q_proj", "k_proj", "v_proj", "gate_proj", "up_proj", "down_proj", "o_proj")):
            continue
        rules.append(rule)
    for i in range(config.num_hidden_layers):
        src, dst = f"model.layers.{i}.", f"layers.{i}."
        for first, count, at in ((0, q_rows, 0), (q_rows, kv_rows, q_rows), (q_rows + kv_rows, kv_rows, q_rows + kv_rows)):
            rules.append(WeightRule(src + "self_attn.qkv_proj.weight", dst + "mixer.qkv_weight", at, count,
                                    source_shape=(width, hidden), source_rows=(first, count)))
            rules.append(WeightRule(src + "self_attn.qkv_proj.bias", dst + "mixer.qkv_bias_vec", at, count,
                                    source_shape=(width,), source_rows=(first, count)))
        rules.append(WeightRule(src + "self_attn.o_proj.weight", dst + "mixer.o_weight", transpose=True))
        rules.append(WeightRule(src + "mlp.gate_up_proj.weight", dst + "feed_forward.gate_up_weight", 0, inter, block=2, period=4,
                                source_shape=(2 * inter, hidden), source_rows=(0, inter)))
        rules.append(WeightRule(src + "mlp.gate_up_proj.weight", dst + "feed_forward.gate_up_weight", 2, inter, block=2, period=4,
                                source_shape=(2 * inter, hidden), source_rows=(inter, inter)))
        rules.append(WeightRule("model.down_stack", dst + "feed_forward.down_weight",
                                source_shape=(config.num_hidden_layers, hidden, inter), source_index=i))
    return tuple(rules)


def test_rules_read_fused_stacked_and_transposed_tensors(tmp_path):
    d = make_model_dir(tmp_path, "B", seed=71, storage_dtype="float32")
    cfg, w = read_weights(d)
    config = Qwen2Config.from_dict(TINY["B"])
    spec = qwen2_spec(config)
    usual = DecoderModel(spec)
    expected = load_weights(usual, d, dtype=torch.float32, device="cpu")
    packed = {n: t for n, t in w.items() if not any(k in n for k in ("q_proj", "k_proj", "v_proj", "gate_proj", "up_proj", "down_proj", "o_proj"))}
    layers = config.num_hidden_layers
    for i in range(layers):
        p = f"model.layers.{i}."
        packed[p + "self_attn.qkv_proj.weight"] = torch.cat([w[p + f"self_attn.{x}_proj.weight"] for x in "qkv"])
        packed[p + "self_attn.qkv_proj.bias"] = torch.cat([w[p + f"self_attn.{x}_proj.bias"] for x in "qkv"])
        packed[p + "self_attn.o_proj.weight"] = w[p + "self_attn.o_proj.weight"].t().contiguous()  # stored [in, out]
        packed[p + "mlp.gate_up_proj.weight"] = torch.cat([w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"]])
    packed["model.down_stack"] = torch.stack([w[f"model.layers.{i}.mlp.down_proj.weight"] for i in range(layers)])
    folder = tmp_path / "packed"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(cfg))
    write_safetensors(folder / "model.safetensors", [(n, t.dtype, tuple(t.shape)) for n, t in packed.items()], iter(packed.items()))
    model = DecoderModel(dataclasses.replace(spec, weight_rules=_packed_rules(config, spec)))
    got = load_weights(model, folder, dtype=torch.float32, device="cpu")
    assert set(got) == set(expected)
    for name, tensor in expected.items():
        assert torch.equal(got[name], tensor), name
    # errors still come in one piece, with the stored shapes the rules expect
    bad = dict(packed)
    bad["model.down_stack"] = bad["model.down_stack"][:, :, :-1].contiguous()
    del bad["model.layers.1.self_attn.qkv_proj.bias"]
    write_safetensors(folder / "model.safetensors", [(n, t.dtype, tuple(t.shape)) for n, t in bad.items()], iter(bad.items()))
    with pytest.raises(WeightsError) as error:
        load_weights(DecoderModel(dataclasses.replace(spec, weight_rules=_packed_rules(config, spec))), folder, dtype=torch.float32, device="cpu")
    assert error.value.missing == ("model.layers.1.self_attn.qkv_proj.bias",)
    assert error.value.wrong_shape[0][0] == "model.down_stack" and tuple(error.value.wrong_shape[0][2]) == (layers, 96, 352)


def test_rules_that_do_not_fit_are_refused_before_any_file_is_read(tmp_path):
    config = Qwen2Config.from_dict(TINY["A"])
    spec = qwen2_spec(config)

    def with_rule(rule):
        rules = tuple(r for r in spec.weight_rules if r.name != "model.layers.0.self_attn.o_proj.weight") + (rule,)
        return DecoderModel(dataclasses.replace(spec, weight_rules=rules))

    name, dest = "model.layers.0.self_attn.o_proj.weight", "layers.0.mixer.o_weight"
    with pytest.raises(ValueError, match="must give source_shape"):
        load_weights(with_rule(WeightRule(name, dest, source_index=0)), tmp_path, dtype=torch.float32, device="cpu")
    with pytest.raises(ValueError, match="wants"):
        load_weights(with_rule(WeightRule(name, dest, source_shape=(3, 64, 65), source_index=1)), tmp_path, dtype=torch.float32, device="cpu")
    with pytest.raises(ValueError, match="outside"):
        load_weights(with_rule(WeightRule(name, dest, source_shape=(2, 64, 64), source_index=2)), tmp_path, dtype=torch.float32, device="cpu")
    assert WeightRule("t", "p", transpose=True).part_shape((3, 5)) == (5, 3)
    assert WeightRule("t", "p", source_index=1, transpose=True, source_rows=(2, 2)).part_shape((4, 3, 5)) == (2, 3)


# ---- what some decoders do around the layers -------------------------------------------------------------------
class LearnedPositions(PositionEncoding):
    """A table with one row per position, added to the embedded tokens."""

    replayable = True

    def __init__(self, positions: int, hidden_size: int) -> None:
        self.positions, self.hidden_size = positions, hidden_size
        self.table = None

    def param_specs(self):
        return {"table": ParamSpec((self.positions, self.hidden_size))}

    def embed(self, ctx):
        return ctx.ops.embedding(self.table, ctx.positions)


def _hooked_spec(config: Qwen2Config):
    spec = qwen2_spec(config)
    rules = spec.weight_rules + (WeightRule("positions.weight", "position_embedding.table"), WeightRule("lm_head.bias", "head.bias"))
    return dataclasses.replace(
        spec, weight_rules=rules, embedding_scale=3.0, head_bias=True, logit_scale=2.0, logit_softcap=1.5,
        position_embedding=PartSpec("toy_learned_positions", {"positions": config.max_position_embeddings, "hidden_size": config.hidden_size}),
    )


@pytest.mark.parametrize("backend,dtype", CASES)
def test_scale_position_embedding_bias_and_soft_cap(tmp_path, backend, dtype):
    register_part("position", "toy_learned_positions", LearnedPositions, replace=True)
    try:
        base = make_model_dir(tmp_path, "A", seed=72)
        cfg, w = read_weights(base)
        config = Qwen2Config.from_dict(TINY["A"])
        g = torch.Generator().manual_seed(3)
        w = dict(w)
        w["positions.weight"] = (torch.randn(config.max_position_embeddings, config.hidden_size, generator=g) * 0.05).to(torch.bfloat16)
        w["lm_head.bias"] = torch.randn(config.vocab_size, generator=g)  # stored in 32-bit: stays 32-bit
        folder = tmp_path / "hooked"
        folder.mkdir()
        (folder / "config.json").write_text(json.dumps(cfg))
        write_safetensors(folder / "model.safetensors", [(n, t.dtype, tuple(t.shape)) for n, t in w.items()], iter(w.items()))
        ops = _ops(backend, dtype)
        model = DecoderModel(_hooked_spec(config))
        assert "head.bias" in model.param_specs() and "position_embedding.table" in model.param_specs()
        params = load_weights(model, folder, dtype=dtype, device=ops.device)
        assert params["head.bias"].dtype == torch.float32
        cache = mlr.make_cache(model, block_size=8, num_blocks=8, max_requests=1)
        runner = ModelRunner(model, cache, ops)
        toks = random_tokens(27, config.vocab_size, 73)
        # the plain model with the same four changes around it
        wd = {k: v.double() for k, v in w.items()}
        x = wd["model.embed_tokens.weight"][torch.tensor(toks)] * 3.0 + wd["positions.weight"][: len(toks)]
        for i in range(config.num_hidden_layers):
            x = plain.decoder_layer(x, torch.arange(len(toks)), wd, i, cfg)
        logits = plain.rms_norm(x, wd["model.norm.weight"], config.rms_norm_eps) @ wd["model.embed_tokens.weight"].t() + wd["lm_head.bias"]
        ref = 1.5 * torch.tanh(logits * 2.0 / 1.5)
        cache.create_request("r")
        got = torch.cat([
            runner.step([StepEntry.of("r", toks[:19], range(19))]).logits,
            runner.step([StepEntry.of("r", toks[19:], range(8))]).logits,
        ]).double().cpu()
        assert float(ref.abs().max()) > 1.3 and float((logits * 2.0).abs().max()) > 3.0, "the cap should matter for this model"
        assert float((got - ref).abs().max()) < (1e-4 if dtype == torch.float32 else 0.06)
        unchanged = plain.forward(toks, {k: v for k, v in w.items() if k not in ("positions.weight", "lm_head.bias")}, cfg)
        assert float((got - unchanged).abs().max()) > 0.3
    finally:
        unregister_part("position", "toy_learned_positions")


# ---- values narrower than keys, or none ------------------------------------------------------------------------------
def test_page_pools_with_other_value_widths():
    wide = PagedKVSpec(2, 16)
    narrow = PagedKVSpec(2, 16, None, 4)
    keys_only = PagedKVSpec(1, 24, None, 0)
    assert (wide.value_dim, narrow.value_dim, keys_only.value_dim) == (16, 4, 0)
    m = CacheManager([wide, narrow, keys_only, narrow], block_size=8, num_blocks=5, max_requests=2, dtype=torch.bfloat16, device="cpu")
    assert [g.sites for g in m.groups] == [(0,), (1, 3), (2,)]
    assert m.groups[1].key.shape == (2, 5, 2, 8, 16) and m.groups[1].value.shape == (2, 5, 2, 4, 8)
    assert m.groups[2].key.shape == (1, 5, 1, 8, 24) and m.groups[2].value.numel() == 0
    assert m.groups[1].storage_bytes() == 2 * 5 * 2 * 8 * (16 + 4) * 2
    assert keys_only.bytes_per_token(2) == 48 and narrow.bytes_per_token(2) == 80
    m.create_request("a")
    lay = m.begin_step([("a", 11)])
    m.commit_step()
    assert all(len(t) == 2 for t in m.get_request("a").tables) and lay.block_tables[2].shape == (1, 2)
    with pytest.raises(ValueError):
        PagedKVSpec(1, 8, None, -1)


# ---- parts that need whole prompts ----------------------------------------------------------------------------------------
class WholePromptAttention(GQAAttention):
    """Attention that, say, could not go on behind a cached prefix."""

    splittable = False


def test_a_part_that_needs_whole_prompts_stops_the_cutting(tmp_path):
    register_part("mixer", "toy_whole_prompt_attention", WholePromptAttention, replace=True)
    try:
        d = make_model_dir(tmp_path, "A", seed=74)
        cfg, w = read_weights(d)
        config = Qwen2Config.from_dict(TINY["A"])
        spec = qwen2_spec(config)
        layers = tuple(dataclasses.replace(l, mixer=PartSpec("toy_whole_prompt_attention", l.mixer.params)) for l in spec.layers)
        model = DecoderModel(dataclasses.replace(spec, layers=layers))
        assert not model.splittable and DecoderModel(spec).splittable
        load_weights(model, d, dtype=torch.float32, device="cpu")
        cache = mlr.make_cache(model, block_size=4, num_blocks=32, max_requests=2)
        runner = ModelRunner(model, cache, TorchOps(torch.float32))
        admission = PageAdmission(cache, max_step_tokens=16)
        with pytest.raises(ValueError, match="whole prompts"):
            ContinuousBatchEngine(scheduler=Scheduler(max_running_requests=2, max_batch_tokens=16, admit=admission.admit),
                                  runner=runner, admission=admission)
        scheduler = Scheduler(max_running_requests=2, max_batch_tokens=16, admit=admission.admit, cut_prompts=False)
        engine = ContinuousBatchEngine(scheduler=scheduler, runner=runner, admission=admission)
        with pytest.raises(ValueError, match="not cut"):
            engine.submit("long", random_tokens(17, 256, 1), max_new_tokens=2)
        a, b = random_tokens(10, 256, 2), random_tokens(9, 256, 3)
        engine.submit("a", a, max_new_tokens=3)
        engine.submit("b", b, max_new_tokens=3)
        first = engine.step()
        assert [len(p.tokens) for p in first.plan.slices] == [10]  # b (9) does not fit beside a and is not cut to 6
        engine.run_until_done()
        assert list(engine.request("a").output) == plain.greedy(a, w, cfg, 3)
        assert list(engine.request("b").output) == plain.greedy(b, w, cfg, 3)
    finally:
        unregister_part("mixer", "toy_whole_prompt_attention")
