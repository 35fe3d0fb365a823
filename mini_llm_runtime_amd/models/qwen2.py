"""Qwen2 dense decoder (`Qwen2ForCausalLM`) as a list of parts.

Every layer is the same pre-norm block: RMSNorm, grouped-query attention with
QKV bias and rotary positions, RMSNorm, SwiGLU
(src/mini_llm_runtime/qwen_model_runner.py:186-218).  Tensor names are the
checkpoint's own (src/mini_llm_runtime/qwen_weights.py:69-119).
"""

from __future__ import annotations

from ..config.qwen2 import Qwen2Config
from ..parts.spec import LayerSpec, ModelSpec, OrderEntry, PartSpec, WeightRule
from .registry import register_architecture


def qwen2_spec(config: Qwen2Config) -> ModelSpec:
    d = config.head_dim
    q_rows = config.num_attention_heads * d
    kv_rows = config.num_key_value_heads * d
    inter = config.intermediate_size
    norm = PartSpec("rms_norm", {"size": config.hidden_size, "eps": config.rms_norm_eps})
    layer = LayerSpec(
        block="pre_norm",
        mixer=PartSpec(
            "gqa_attention",
            {
                "hidden_size": config.hidden_size,
                "num_heads": config.num_attention_heads,
                "num_kv_heads": config.num_key_value_heads,
                "head_dim": d,
                "qkv_bias": True,  # always present: qwen_weights.py:77, 81, 85
                "o_bias": False,  # never present: qwen_weights.py:87-89
                "position": PartSpec("rotary", {"head_dim": d, "theta": config.rope_theta}),
            },
        ),
        feed_forward=PartSpec(
            "swiglu", {"hidden_size": config.hidden_size, "intermediate_size": inter}
        ),
        norms={"input": norm, "post_mixer": norm},
    )
    rules: list[WeightRule] = [WeightRule("model.embed_tokens.weight", "embed.weight")]
    for i in range(config.num_hidden_layers):
        src = f"model.layers.{i}."
        dst = f"layers.{i}."
        rules += [
            WeightRule(src + "input_layernorm.weight", dst + "norm_input.weight"),
            WeightRule(src + "self_attn.q_proj.weight", dst + "mixer.qkv_weight", 0, q_rows),
            WeightRule(src + "self_attn.k_proj.weight", dst + "mixer.qkv_weight", q_rows, kv_rows),
            WeightRule(src + "self_attn.v_proj.weight", dst + "mixer.qkv_weight", q_rows + kv_rows, kv_rows),
            WeightRule(src + "self_attn.q_proj.bias", dst + "mixer.qkv_bias_vec", 0, q_rows),
            WeightRule(src + "self_attn.k_proj.bias", dst + "mixer.qkv_bias_vec", q_rows, kv_rows),
            WeightRule(src + "self_attn.v_proj.bias", dst + "mixer.qkv_bias_vec", q_rows + kv_rows, kv_rows),
            WeightRule(src + "self_attn.o_proj.weight", dst + "mixer.o_weight"),
            WeightRule(src + "post_attention_layernorm.weight", dst + "norm_post_mixer.weight"),
            # gate and up rows woven in pairs (g g u u g g u u ...): the product's epilogue
            # then holds a gate sum beside its up sum and applies SwiGLU without another kernel
            WeightRule(src + "mlp.gate_proj.weight", dst + "feed_forward.gate_up_weight", 0, inter, block=2, period=4),
            WeightRule(src + "mlp.up_proj.weight", dst + "feed_forward.gate_up_weight", 2, inter, block=2, period=4),
            WeightRule(src + "mlp.down_proj.weight", dst + "feed_forward.down_weight"),
        ]
    rules.append(WeightRule("model.norm.weight", "final_norm.weight"))
    if config.tie_word_embeddings:
        # tied checkpoints usually do not store the head; one that does must repeat the
        # embedding (qwen_weights.py:114-119)
        rules.append(WeightRule("lm_head.weight", "embed.weight", optional=True, must_equal="embed.weight"))
    else:
        rules.append(WeightRule("lm_head.weight", "head.weight"))
    return ModelSpec(
        architecture=config.architecture,
        vocab_size=config.vocab_size,
        hidden_size=config.hidden_size,
        max_position_embeddings=config.max_position_embeddings,
        layers=tuple(layer for _ in range(config.num_hidden_layers)),
        order=tuple(OrderEntry(i) for i in range(config.num_hidden_layers)),
        final_norm=norm,
        tie_word_embeddings=config.tie_word_embeddings,
        weight_rules=tuple(rules),
    )


register_architecture(Qwen2Config.architecture, Qwen2Config, qwen2_spec, replace=True)
