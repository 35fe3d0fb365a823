"""Configuration, registry, weight loading errors and the random-weights mode (CPU)."""

from __future__ import annotations

import json

import pytest
import torch

import mini_llm_runtime_amd as mlr
from helpers import TINY_A, TINY_B, make_model_dir, read_weights
from mini_llm_runtime_amd.config import ConfigError, Qwen2Config
from mini_llm_runtime_amd.models import ARCHITECTURES, build_model, config_from_dict
from mini_llm_runtime_amd.weights import SafetensorsFile, WeightsError, load_weights, save_state_dict


def test_config_reads_its_own_keys():
    c = Qwen2Config.from_dict(TINY_B)
    assert (c.hidden_size, c.num_attention_heads, c.head_dim, c.gqa_group_size) == (96, 3, 32, 3)
    assert c.tie_word_embeddings is False and c.rms_norm_eps == 1e-5
    a = Qwen2Config.from_dict(TINY_A)
    assert a.head_dim == 16  # derived: hidden_size // num_attention_heads (qwen_config.py:46-48 of the reference)
    assert Qwen2Config.from_dict(a.to_dict()) == a


@pytest.mark.parametrize(
    "change,match",
    [
        ({"model_type": "llama"}, "model_type"),
        ({"rope_scaling": {"type": "yarn"}}, "rope_scaling"),
        ({"use_sliding_window": True}, "sliding"),
        ({"hidden_act": "gelu"}, "silu"),
        ({"num_key_value_heads": 3}, "multiple"),
        ({"vocab_size": 0}, "positive"),
        ({"rms_norm_eps": 0}, "positive"),
        ({"head_dim": 15}, "even"),
    ],
)
def test_config_refuses_unsupported_variants(change, match):
    with pytest.raises(ConfigError, match=match):
        Qwen2Config.from_dict({**TINY_A, **change})


def test_config_missing_keys_are_listed():
    data = {k: v for k, v in TINY_A.items() if k not in ("rope_theta", "vocab_size")}
    with pytest.raises(ConfigError, match="vocab_size, rope_theta|rope_theta.*vocab_size|vocab_size.*rope_theta"):
        Qwen2Config.from_dict(data)


def test_registry_chooses_by_architecture_name():
    assert "Qwen2ForCausalLM" in ARCHITECTURES
    assert isinstance(config_from_dict(TINY_A), Qwen2Config)
    with pytest.raises(ConfigError, match="unknown architecture 'NopeForCausalLM'.*Qwen2ForCausalLM"):
        config_from_dict({**TINY_A, "architectures": ["NopeForCausalLM"]})
    only_type = {k: v for k, v in TINY_A.items() if k != "architectures"}
    assert isinstance(config_from_dict(only_type), Qwen2Config)


def test_model_spec_takes_every_size_from_the_config():
    model = build_model(Qwen2Config.from_dict(TINY_B))
    specs = model.param_specs()
    assert specs["layers.2.mixer.qkv_weight"].shape == ((3 + 2) * 32, 96)
    assert specs["layers.0.feed_forward.gate_up_weight"].shape == (2 * 352, 96)
    assert specs["head.weight"].shape == (517, 96)
    assert "head.weight" not in build_model(Qwen2Config.from_dict(TINY_A)).param_specs()
    assert len(model.site_cache_specs()) == 3


def test_a_head_size_no_kernel_runs_is_refused_when_the_model_is_built():
    """Sizes that only slower kernels take build fine (a head size of 20, of 264 would not);
    a head size beyond what any attention kernel keeps in registers is refused at once."""
    ok = Qwen2Config.from_dict({**TINY_A, "head_dim": 256})
    assert build_model(ok).layers[0].mixer.head_dim == 256
    too_wide = Qwen2Config.from_dict({**TINY_A, "head_dim": 272})
    with pytest.raises(ValueError, match="head_dim 272.*up to 256"):
        build_model(too_wide)


def test_an_odd_intermediate_size_is_refused_when_the_model_is_built():
    """Gate and up rows are woven in pairs for the SwiGLU epilogue: an odd number of them has no such
    layout, and the feed-forward says so instead of computing something else."""
    with pytest.raises(ValueError, match="intermediate size even"):
        build_model(Qwen2Config.from_dict({**TINY_A, "intermediate_size": 129}))


def test_random_model_is_seeded_and_loads(tmp_path):
    d1 = make_model_dir(tmp_path / "x", "A", seed=5)
    d2 = make_model_dir(tmp_path / "y", "A", seed=5)
    d3 = make_model_dir(tmp_path / "z", "A", seed=6)
    _, w1 = read_weights(d1)
    _, w2 = read_weights(d2)
    _, w3 = read_weights(d3)
    assert all(torch.equal(w1[k], w2[k]) for k in w1)
    assert not torch.equal(w1["model.norm.weight"], w3["model.norm.weight"])
    assert "lm_head.weight" not in w1  # tied checkpoints do not store the head
    assert w1["model.norm.weight"].dtype == torch.bfloat16
    assert abs(float(w1["model.norm.weight"].float().mean()) - 1.0) < 0.05
    assert abs(float(w1["model.embed_tokens.weight"].float().std()) - 0.02) < 0.005
    config, model = mlr.load_model(d1, dtype="float32", device="cpu")
    assert model.embed_weight.dtype == torch.float32 and model.head_weight is model.embed_weight
    q = w1["model.layers.1.self_attn.q_proj.weight"].float()
    k = w1["model.layers.1.self_attn.k_proj.weight"].float()
    fused = model.layers[1].mixer.qkv_weight
    assert torch.equal(fused[:64], q) and torch.equal(fused[64:96], k)


def test_dtype_rules(tmp_path):
    """bfloat16 stays bfloat16; a vector stored in 32-bit stays 32-bit; matrices take the engine's dtype."""
    d = make_model_dir(tmp_path, "A", seed=1)
    cfg, w = read_weights(d)
    w = dict(w)
    w["model.norm.weight"] = w["model.norm.weight"].float()
    w["model.layers.0.self_attn.o_proj.weight"] = w["model.layers.0.self_attn.o_proj.weight"].float()
    save_state_dict(d / "model.safetensors", w)
    _, model = mlr.load_model(d, dtype="bfloat16", device="cpu")
    assert model.final_norm.weight.dtype == torch.float32
    assert model.layers[0].norm_input.weight.dtype == torch.bfloat16
    assert model.layers[0].mixer.o_weight.dtype == torch.bfloat16
    assert model.embed_weight.dtype == torch.bfloat16


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = make_model_dir(tmp_path, "B", seed=1)
    cfg, w = read_weights(d)
    w = dict(w)
    del w["model.layers.1.mlp.up_proj.weight"]
    del w["lm_head.weight"]
    w["model.layers.0.self_attn.o_proj.bias"] = torch.zeros(96)
    w["model.layers.2.self_attn.k_proj.weight"] = torch.zeros(32, 95)
    save_state_dict(d / "model.safetensors", w)
    model = build_model(config_from_dict(cfg))
    with pytest.raises(WeightsError) as info:
        load_weights(model, d, dtype=torch.float32, device="cpu")
    e = info.value
    assert set(e.missing) == {"model.layers.1.mlp.up_proj.weight", "lm_head.weight"}
    assert e.unexpected == ("model.layers.0.self_attn.o_proj.bias",)
    assert e.wrong_shape == (("model.layers.2.self_attn.k_proj.weight", (32, 95), (32, 96)),)
    text = str(e)
    for name in (*e.missing, *e.unexpected, "model.layers.2.self_attn.k_proj.weight"):
        assert name in text


def test_tied_head_stored_twice_must_repeat_the_embedding(tmp_path):
    d = make_model_dir(tmp_path, "A", seed=1)
    cfg, w = read_weights(d)
    w = dict(w)
    w["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    save_state_dict(d / "model.safetensors", w)
    mlr.load_model(d, dtype="float32", device="cpu")
    w["lm_head.weight"][3, 3] += 1
    save_state_dict(d / "model.safetensors", w)
    with pytest.raises(WeightsError, match="lm_head.weight"):
        mlr.load_model(d, dtype="float32", device="cpu")


def test_sharded_checkpoint_with_index(tmp_path):
    d = make_model_dir(tmp_path, "A", seed=1)
    cfg, w = read_weights(d)
    names = sorted(w)
    half = len(names) // 2
    shards = {"model-00001-of-00002.safetensors": names[:half], "model-00002-of-00002.safetensors": names[half:]}
    (d / "model.safetensors").unlink()
    for shard, keys in shards.items():
        save_state_dict(d / shard, {k: w[k] for k in keys})
    with pytest.raises(FileNotFoundError, match="index"):
        mlr.load_model(d, dtype="float32", device="cpu")
    (d / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {k: s for s, ks in shards.items() for k in ks}}))
    _, model = mlr.load_model(d, dtype="float32", device="cpu")
    assert torch.equal(model.final_norm.weight, w["model.norm.weight"].float())


def test_safetensors_reader_rejects_garbage(tmp_path):
    p = tmp_path / "bad.safetensors"
    p.write_bytes(b"\x10\x00\x00\x00\x00\x00\x00\x00not json at all!")
    with pytest.raises(ValueError):
        SafetensorsFile(p)
    p.write_bytes(b"\x01")
    with pytest.raises(ValueError):
        SafetensorsFile(p)


def test_no_cpu_path_in_the_product():
    from mini_llm_runtime_amd.kernels.ops import HipOps, KernelError

    with pytest.raises(KernelError, match="no CPU path"):
        HipOps(torch.float32, "cpu")
