"""A plain, slow Qwen2 decoder: whole sequences, no cache, one function per part.

Written from the formulas of the reference (file:line cited per function, paths
relative to the reference's root).  It shares no code with the engine: it only
uses torch tensor arithmetic, runs on the CPU and recomputes everything for every
call.  All arithmetic is done in the dtype of the tensors it is given (the tests
pass float64 or float32), so the rounding steps the reference inserts when its
model dtype is 16-bit are no-ops here.
"""

from __future__ import annotations

import math
from typing import Mapping, Sequence

import torch


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """`weight * x * rsqrt(mean(x^2, -1) + eps)`; no centring, no bias, weight as is.

    src/mini_llm_runtime/qwen_model_runner.py:22-26
    """
    variance = x.pow(2).mean(dim=-1, keepdim=True)
    return weight * (x * torch.rsqrt(variance + eps))


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """`cat(-x[d/2:], x[:d/2])`: dims j and j+d/2 are a pair (half-split layout).

    src/mini_llm_runtime/qwen_model_runner.py:34-36
    """
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def rope_angles(positions: torch.Tensor, head_dim: int, theta: float) -> torch.Tensor:
    """Angles `pos * theta^(-2j/d)`, j = 0..d/2-1, repeated for both halves: [S, d].

    src/mini_llm_runtime/qwen_model_runner.py:45-55
    """
    exponents = torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim
    inv_freq = 1.0 / (float(theta) ** exponents)
    freqs = positions.to(torch.float64)[:, None] * inv_freq[None, :]
    return torch.cat((freqs, freqs), dim=-1)


def apply_rope(x: torch.Tensor, positions: torch.Tensor, theta: float) -> torch.Tensor:
    """`x * cos + rotate_half(x) * sin` for x of shape [heads, S, d].

    src/mini_llm_runtime/qwen_model_runner.py:56-61
    """
    angles = rope_angles(positions, x.shape[-1], theta)
    cos = angles.cos().to(x.dtype)[None]
    sin = angles.sin().to(x.dtype)[None]
    return x * cos + rotate_half(x) * sin


def repeat_kv(x: torch.Tensor, repeats: int) -> torch.Tensor:
    """[Hkv, S, d] -> [Hkv*repeats, S, d]; query head h reads KV head h // repeats.

    src/mini_llm_runtime/qwen_model_runner.py:64-72
    """
    if repeats == 1:
        return x
    heads, seq, dim = x.shape
    return x[:, None].expand(heads, repeats, seq, dim).reshape(heads * repeats, seq, dim)


def causal_attention(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    *,
    scale: float | None = None,
    causal: bool = True,
    window: int | None = None,
) -> torch.Tensor:
    """softmax(q k^T / sqrt(d) + mask) v for q [Hq,S,d], k/v [Hkv,S,d] -> [Hq,S,d].

    Scores, mask, softmax and the weighted sum follow
    src/mini_llm_runtime/qwen_model_runner.py:138-139, 157-177 (a key is visible when
    its index is not larger than the query's).  `window`, when given, additionally
    hides keys more than `window - 1` positions behind the query; the reference has
    no such option (qwen_config.py:65-77 never reads the window keys).
    """
    hq, seq, dim = query.shape
    group = hq // key.shape[0]
    key = repeat_kv(key, group)
    value = repeat_kv(value, group)
    if scale is None:
        scale = 1.0 / math.sqrt(dim)
    scores = torch.matmul(query, key.transpose(-2, -1)) * scale
    if causal:
        q_idx = torch.arange(seq)[:, None]
        k_idx = torch.arange(key.shape[1])[None, :]
        hidden = k_idx > q_idx
        if window is not None:
            hidden = hidden | (k_idx < q_idx - (window - 1))
        scores = scores.masked_fill(hidden[None], float("-inf"))
    probabilities = torch.softmax(scores, dim=-1)
    return torch.matmul(probabilities, value)


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """`x W^T + b` with W stored [out_features, in_features].

    src/mini_llm_runtime/qwen_model_runner.py:88-102 (F.linear semantics)
    """
    y = x @ weight.transpose(0, 1)
    return y if bias is None else y + bias


def attention_block(
    x: torch.Tensor,
    positions: torch.Tensor,
    w: Mapping[str, torch.Tensor],
    prefix: str,
    *,
    num_heads: int,
    num_kv_heads: int,
    head_dim: int,
    theta: float,
) -> torch.Tensor:
    """Project, split into heads, rotate q and k, attend, merge heads, o_proj (no bias).

    src/mini_llm_runtime/qwen_model_runner.py:75-183
    """
    seq = x.shape[0]
    q = linear(x, w[prefix + "q_proj.weight"], w[prefix + "q_proj.bias"])
    k = linear(x, w[prefix + "k_proj.weight"], w[prefix + "k_proj.bias"])
    v = linear(x, w[prefix + "v_proj.weight"], w[prefix + "v_proj.bias"])
    q = q.reshape(seq, num_heads, head_dim).transpose(0, 1)
    k = k.reshape(seq, num_kv_heads, head_dim).transpose(0, 1)
    v = v.reshape(seq, num_kv_heads, head_dim).transpose(0, 1)
    q = apply_rope(q, positions, theta)
    k = apply_rope(k, positions, theta)
    per_head = causal_attention(q, k, v)
    merged = per_head.transpose(0, 1).reshape(seq, num_heads * head_dim)
    return linear(merged, w[prefix + "o_proj.weight"])


def swiglu(x: torch.Tensor, w: Mapping[str, torch.Tensor], prefix: str) -> torch.Tensor:
    """`down(silu(gate(x)) * up(x))`, silu(z) = z * sigmoid(z), no biases.

    src/mini_llm_runtime/qwen_model_runner.py:215-217
    """
    gate = linear(x, w[prefix + "gate_proj.weight"])
    up = linear(x, w[prefix + "up_proj.weight"])
    return linear(gate * torch.sigmoid(gate) * up, w[prefix + "down_proj.weight"])


def decoder_layer(
    x: torch.Tensor,
    positions: torch.Tensor,
    w: Mapping[str, torch.Tensor],
    index: int,
    cfg: Mapping[str, object],
) -> torch.Tensor:
    """Pre-norm block: x + attn(norm(x)), then x + mlp(norm(x)).

    src/mini_llm_runtime/qwen_model_runner.py:198-218
    """
    p = f"model.layers.{index}."
    eps = float(cfg["rms_norm_eps"])
    heads = int(cfg["num_attention_heads"])
    head_dim = int(cfg.get("head_dim") or int(cfg["hidden_size"]) // heads)
    h = rms_norm(x, w[p + "input_layernorm.weight"], eps)
    x = x + attention_block(
        h,
        positions,
        w,
        p + "self_attn.",
        num_heads=heads,
        num_kv_heads=int(cfg["num_key_value_heads"]),
        head_dim=head_dim,
        theta=float(cfg["rope_theta"]),
    )
    h = rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
    return x + swiglu(h, w, p + "mlp.")


def forward(
    token_ids: Sequence[int],
    weights: Mapping[str, torch.Tensor],
    cfg: Mapping[str, object],
    *,
    dtype: torch.dtype = torch.float64,
    position_offset: int = 0,
) -> torch.Tensor:
    """Logits [S, vocab] of one whole sequence, every position, nothing cached.

    Embedding gather, the layers in order, final norm, then the head: the embedding
    matrix again when `tie_word_embeddings`, else `lm_head.weight`
    (src/mini_llm_runtime/qwen_model_runner.py:263-290; the untied head is this
    build's addition, the reference refuses it at qwen_config.py:43-44).
    `position_offset` shifts every position by a constant; it exists for the
    invariance test (only distances between positions may matter).
    """
    w = {name: t.to(dtype) for name, t in weights.items()}
    ids = torch.as_tensor(list(token_ids), dtype=torch.long)
    positions = torch.arange(len(ids)) + position_offset
    x = w["model.embed_tokens.weight"][ids]
    for index in range(int(cfg["num_hidden_layers"])):
        x = decoder_layer(x, positions, w, index, cfg)
    x = rms_norm(x, w["model.norm.weight"], float(cfg["rms_norm_eps"]))
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return linear(x, head)


def greedy(
    prompt: Sequence[int],
    weights: Mapping[str, torch.Tensor],
    cfg: Mapping[str, object],
    max_new_tokens: int,
    *,
    dtype: torch.dtype = torch.float64,
) -> list[int]:
    """Recompute-everything greedy decoding (argmax, first maximum wins).

    src/mini_llm_runtime/generation.py:84-104; tests/test_generation.py:14-52 of the
    reference compare cached generation against exactly this loop.
    """
    tokens = list(prompt)
    out: list[int] = []
    for _ in range(max_new_tokens):
        logits = forward(tokens, weights, cfg, dtype=dtype)
        nxt = int(torch.argmax(logits[-1]).item())
        out.append(nxt)
        tokens.append(nxt)
    return out


def temperature_probabilities(logits: torch.Tensor, temperature: float) -> torch.Tensor:
    """softmax(logits / temperature) in float64 (this build's sampler; the reference is greedy only,
    src/mini_llm_runtime/engine.py:222)."""
    return torch.softmax(logits.to(torch.float64) / temperature, dim=-1)
