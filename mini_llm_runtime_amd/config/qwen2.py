"""The Qwen2 dense decoder's configuration (`Qwen2ForCausalLM`, model_type `qwen2`)."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar, Mapping

from .model_config import (
    ConfigError,
    ModelConfig,
    positive_float,
    positive_int,
    require_keys,
)


@dataclass(frozen=True)
class Qwen2Config(ModelConfig):
    """Sizes and constants of a Qwen2 decoder, from config.json.

    Keys and checks follow src/mini_llm_runtime/qwen_config.py:9-93 of the reference:
    the same eleven required keys, `model_type == "qwen2"`, no `rope_scaling`, all
    sizes positive, query heads a multiple of KV heads, `hidden_act == "silu"`.
    Beyond the reference: `head_dim` is read when present (default
    hidden_size // num_attention_heads, qwen_config.py:46-48), and
    `tie_word_embeddings=false` is accepted (the reference refuses it at
    qwen_config.py:43-44) and selects a separate `lm_head.weight`.  A config that
    switches the sliding window on is refused: the reference never reads those keys
    (qwen_config.py:65-77), so there is no behaviour to match.
    """

    architecture: ClassVar[str] = "Qwen2ForCausalLM"
    model_type: ClassVar[str] = "qwen2"

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    hidden_act: str
    tie_word_embeddings: bool
    head_dim: int = 0

    def __post_init__(self) -> None:
        for name in (
            "vocab_size",
            "hidden_size",
            "intermediate_size",
            "num_hidden_layers",
            "num_attention_heads",
            "num_key_value_heads",
            "max_position_embeddings",
        ):
            if getattr(self, name) <= 0:
                raise ConfigError(f"Qwen2Config.{name} must be > 0")
        if self.head_dim == 0:
            if self.hidden_size % self.num_attention_heads != 0:
                raise ConfigError(
                    "hidden_size must be a multiple of num_attention_heads when head_dim is not given"
                )
            object.__setattr__(self, "head_dim", self.hidden_size // self.num_attention_heads)
        if self.head_dim <= 0 or self.head_dim % 2 != 0:
            raise ConfigError("head_dim must be positive and even (rotary pairs)")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError("num_attention_heads must be a multiple of num_key_value_heads")
        if not self.rms_norm_eps > 0 or not self.rope_theta > 0:
            raise ConfigError("rms_norm_eps and rope_theta must be > 0")
        if self.hidden_act != "silu":
            raise ConfigError(f"hidden_act must be 'silu' (SwiGLU), found {self.hidden_act!r}")

    @property
    def gqa_group_size(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "Qwen2Config":
        if data.get("model_type", cls.model_type) != cls.model_type:
            raise ConfigError(
                f"Qwen2Config needs model_type={cls.model_type!r}, found {data.get('model_type')!r}"
            )
        if data.get("rope_scaling") is not None:
            raise ConfigError("rope_scaling is not supported for Qwen2 (must be absent or null)")
        if data.get("use_sliding_window"):
            raise ConfigError("use_sliding_window=true is not supported for Qwen2")
        require_keys(
            data,
            (
                "vocab_size",
                "hidden_size",
                "intermediate_size",
                "num_hidden_layers",
                "num_attention_heads",
                "num_key_value_heads",
                "max_position_embeddings",
                "rms_norm_eps",
                "rope_theta",
                "hidden_act",
                "tie_word_embeddings",
            ),
            "Qwen2Config",
        )
        head_dim = data.get("head_dim")
        return cls(
            vocab_size=positive_int(data, "vocab_size"),
            hidden_size=positive_int(data, "hidden_size"),
            intermediate_size=positive_int(data, "intermediate_size"),
            num_hidden_layers=positive_int(data, "num_hidden_layers"),
            num_attention_heads=positive_int(data, "num_attention_heads"),
            num_key_value_heads=positive_int(data, "num_key_value_heads"),
            max_position_embeddings=positive_int(data, "max_position_embeddings"),
            rms_norm_eps=positive_float(data, "rms_norm_eps"),
            rope_theta=positive_float(data, "rope_theta"),
            hidden_act=str(data["hidden_act"]),
            tie_word_embeddings=bool(data["tie_word_embeddings"]),
            head_dim=0 if head_dim is None else positive_int(data, "head_dim"),
        )
