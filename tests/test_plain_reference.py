"""Pins of the plain implementation beside the reference's text: vectors that the
reference's own tests hold, special cases that reduce to a library routine, and
invariants.  Each is chosen so that a plausible mistake fails it."""

from __future__ import annotations

import math

import pytest
import torch

import plain_qwen2 as plain
from helpers import make_model_dir, random_tokens, read_weights


def test_rotate_half_vector():
    # reference tests/test_manual_qwen_attention.py:11-14 (a wrong sign or an interleaved pairing fails)
    assert plain.rotate_half(torch.tensor([1.0, 2.0, 3.0, 4.0])).tolist() == [-3.0, -4.0, 1.0, 2.0]


def test_repeat_kv_order():
    # reference tests/test_manual_qwen_attention.py:17-21: adjacent query heads share a KV head
    x = torch.tensor([10.0, 20.0]).view(2, 1, 1)
    assert plain.repeat_kv(x, 3).flatten().tolist() == [10, 10, 10, 20, 20, 20]


def test_rope_position_zero_is_identity_and_norm_preserving():
    # reference tests/test_manual_qwen_attention.py:35-42
    x = torch.randn(3, 5, 16, dtype=torch.float64)
    pos = torch.tensor([0, 1, 7, 100, 4000])
    y = plain.apply_rope(x, pos, 10000.0)
    assert torch.equal(y[:, 0], x[:, 0])
    # each (j, j + d/2) pair is rotated: its norm is kept
    pair = lambda t: t[..., :8] ** 2 + t[..., 8:] ** 2
    torch.testing.assert_close(pair(y), pair(x))


def test_rope_scores_depend_on_distance_only():
    q = torch.randn(1, 1, 32, dtype=torch.float64)
    k = torch.randn(1, 1, 32, dtype=torch.float64)
    def score(m, n):
        return float((plain.apply_rope(q, torch.tensor([m]), 1e6) * plain.apply_rope(k, torch.tensor([n]), 1e6)).sum())
    assert score(5, 2) == pytest.approx(score(105, 102), abs=1e-9)
    assert score(5, 2) != pytest.approx(score(5, 3), abs=1e-6)
    # the sign of the rotation: q at m against k at n equals the unrotated q against k rotated by n - m
    assert score(3, 0) == pytest.approx(float((q * plain.apply_rope(k, torch.tensor([-3]), 1e6)).sum()), abs=1e-9)


def test_rope_theta_enters_through_inverse_frequencies():
    ang = plain.rope_angles(torch.tensor([1]), 8, 100.0)[0]
    expect = [100.0 ** (-2 * j / 8) for j in range(4)]
    assert ang.tolist() == pytest.approx(expect + expect)


def test_rms_norm_vectors():
    # reference tests/test_manual_qwen_decoder_layer.py:8-18
    rms = math.sqrt(12.5)
    got = plain.rms_norm(torch.tensor([3.0, 4.0]), torch.tensor([2.0, 0.5]), 0.0)
    assert got.tolist() == pytest.approx([2 * 3 / rms, 0.5 * 4 / rms])
    ones = plain.rms_norm(torch.ones(6), torch.ones(6), 0.0)
    assert ones.tolist() == [1.0] * 6  # LayerNorm would give zeros; a "1 + w" weight would give 2
    x = torch.randn(4, 10, dtype=torch.float64)
    torch.testing.assert_close(plain.rms_norm(3 * x, torch.ones(10, dtype=torch.float64), 0.0),
                               plain.rms_norm(x, torch.ones(10, dtype=torch.float64), 0.0))


def test_attention_reduces_to_library_routine():
    # no rotation, full heads: torch's scaled_dot_product_attention(is_causal=True)
    q, k, v = (torch.randn(3, 11, 8, dtype=torch.float64) for _ in range(3))
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
    torch.testing.assert_close(plain.causal_attention(q, k, v), ref)
    # one token of context: the output is v exactly
    torch.testing.assert_close(plain.causal_attention(q[:, :1], k[:, :1], v[:, :1]), v[:, :1])
    # MQA: every head reads the same KV head
    out = plain.causal_attention(q, k[:1], v[:1])
    ref = torch.nn.functional.scaled_dot_product_attention(q, k[:1].expand(3, -1, -1), v[:1].expand(3, -1, -1), is_causal=True)
    torch.testing.assert_close(out, ref)


def test_attention_window_hides_old_keys():
    q, k, v = (torch.randn(1, 9, 4, dtype=torch.float64) for _ in range(3))
    full = plain.causal_attention(q, k, v)
    assert torch.allclose(plain.causal_attention(q, k, v, window=9), full)
    w1 = plain.causal_attention(q, k, v, window=1)
    torch.testing.assert_close(w1, v)  # a window of one sees only the token itself
    w3 = plain.causal_attention(q, k, v, window=3)
    torch.testing.assert_close(w3[:, 8:9], plain.causal_attention(q[:, 6:9], k[:, 6:9], v[:, 6:9])[:, 2:3])


def test_swiglu_identity_weights():
    # reference tests/test_manual_qwen_decoder_layer.py:21-36: silu(x) * 2x through identity weights
    eye = torch.eye(3, dtype=torch.float64)
    w = {"m.gate_proj.weight": eye, "m.up_proj.weight": 2 * eye, "m.down_proj.weight": eye}
    x = torch.tensor([[-1.0, 0.5, 2.0]], dtype=torch.float64)
    torch.testing.assert_close(plain.swiglu(x, w, "m."), torch.nn.functional.silu(x) * 2 * x)


def test_linear_layout_is_out_by_in():
    w = torch.arange(6.0).view(2, 3)  # [out=2, in=3]
    assert plain.linear(torch.tensor([[1.0, 0.0, 0.0]]), w).tolist() == [[0.0, 3.0]]


def test_embedding_and_tied_head_use_one_matrix(tmp_path):
    # reference tests/test_manual_qwen_model_runner.py:7-16; untied must differ
    d = make_model_dir(tmp_path, "A", seed=2)
    cfg, w = read_weights(d)
    toks = random_tokens(6, cfg["vocab_size"], 3)
    tied = plain.forward(toks, w, cfg)
    other = dict(w)
    other["lm_head.weight"] = torch.randn_like(w["model.embed_tokens.weight"].float())
    cfg2 = dict(cfg, tie_word_embeddings=False)
    assert not torch.allclose(plain.forward(toks, other, cfg2), tied)
    other["lm_head.weight"] = w["model.embed_tokens.weight"]
    torch.testing.assert_close(plain.forward(toks, other, cfg2), tied)


@pytest.mark.parametrize("which", ["A", "B"])
def test_causality_and_prefix_consistency(tmp_path, which):
    """Logits at position i depend on tokens 0..i only: a longer sequence reproduces a shorter one."""
    d = make_model_dir(tmp_path, which, seed=4)
    cfg, w = read_weights(d)
    toks = random_tokens(20, cfg["vocab_size"], 5)
    full = plain.forward(toks, w, cfg)
    torch.testing.assert_close(plain.forward(toks[:13], w, cfg), full[:13])
    changed = list(toks)
    changed[15] = (changed[15] + 1) % cfg["vocab_size"]
    again = plain.forward(changed, w, cfg)
    torch.testing.assert_close(again[:15], full[:15])
    assert not torch.allclose(again[15:], full[15:])


def test_shift_of_all_positions_changes_nothing(tmp_path):
    """Only distances between positions count."""
    d = make_model_dir(tmp_path, "B", seed=6)
    cfg, w = read_weights(d)
    toks = random_tokens(12, cfg["vocab_size"], 7)
    torch.testing.assert_close(plain.forward(toks, w, cfg, position_offset=37), plain.forward(toks, w, cfg), atol=1e-9, rtol=0)


def _reference_fixture():
    """The reference's own tiny fixture (tests/test_qwen_weights.py:9-65): vocab 5, hidden 4,
    2 layers, 2 heads / 1 KV head, head_dim 2; weights from torch.randn with seed 7, drawn in
    the order of its `tiny_state_dict`."""
    cfg = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2",
               vocab_size=5, hidden_size=4, intermediate_size=6, num_hidden_layers=2, num_attention_heads=2,
               num_key_value_heads=1, max_position_embeddings=8, rms_norm_eps=1e-6, rope_theta=10000.0,
               hidden_act="silu", tie_word_embeddings=True)
    g = torch.Generator().manual_seed(7)
    def r(*s):
        return torch.randn(*s, generator=g)
    w = {"model.embed_tokens.weight": r(5, 4), "model.norm.weight": r(4)}
    for i in range(2):
        p = f"model.layers.{i}."
        w.update({p + "input_layernorm.weight": r(4), p + "post_attention_layernorm.weight": r(4),
                  p + "self_attn.q_proj.weight": r(4, 4), p + "self_attn.q_proj.bias": r(4),
                  p + "self_attn.k_proj.weight": r(2, 4), p + "self_attn.k_proj.bias": r(2),
                  p + "self_attn.v_proj.weight": r(2, 4), p + "self_attn.v_proj.bias": r(2),
                  p + "self_attn.o_proj.weight": r(4, 4), p + "mlp.gate_proj.weight": r(6, 4),
                  p + "mlp.up_proj.weight": r(6, 4), p + "mlp.down_proj.weight": r(4, 6)})
    return cfg, w


@pytest.mark.parametrize("backend", ["double", pytest.param("hip", marks=pytest.mark.gpu)])
def test_reference_tiny_fixture_cached_equals_recomputed(tmp_path, backend):
    """What the reference asserts on this fixture (tests/test_generation.py:31-52): generation
    from the cache gives the tokens AND the per-step logits (atol 1e-5) of the loop that
    recomputes everything, with its counts (3 new tokens: 3 prompt tokens, 2 decode steps, 5
    cached).  Here the cached side is the engine (32-bit), the other the plain implementation."""
    import json

    import mini_llm_runtime_amd as mlr
    from kernel_doubles import TorchOps
    from mini_llm_runtime_amd.engine import ModelRunner
    from mini_llm_runtime_amd.weights.safetensors_io import write_safetensors

    cfg, w = _reference_fixture()
    folder = tmp_path / "fixture"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(cfg))
    write_safetensors(folder / "model.safetensors", [(n, t.dtype, tuple(t.shape)) for n, t in w.items()], iter(w.items()))
    if backend == "double":
        ops = TorchOps(torch.float32, "cpu")
    else:
        from mini_llm_runtime_amd.kernels.ops import HipOps

        ops = HipOps(torch.float32, "cuda")
    _, model = mlr.load_model(folder, dtype=torch.float32, device=ops.device)
    cache = mlr.make_cache(model, block_size=2, num_blocks=4, max_requests=1)
    out = mlr.greedy_generate(ModelRunner(model, cache, ops), [1, 2, 3], max_new_tokens=3, return_step_logits=True)
    seq, expected = [1, 2, 3], []
    for i in range(3):
        logits = plain.forward(seq, w, cfg)[-1]
        assert float((out.step_logits[i].double().cpu() - logits).abs().max()) < 1e-5, f"step {i}"
        expected.append(int(torch.argmax(logits)))
        seq.append(expected[-1])
    assert list(out.generated_token_ids) == expected == plain.greedy([1, 2, 3], w, cfg, 3)
    assert (out.prefill_tokens, out.decode_steps, out.cache_length, out.stopped_by_eos) == (3, 2, 5, False)
