"""What the kernel library takes, as far as a model can be checked against it before any
kernel exists: parts that are bound to these kernels ask here when they are constructed, so a
configuration that cannot run is refused when the model is built, not at its first step.
(The reference refuses what it cannot run when the config is read,
src/mini_llm_runtime/qwen_config.py:23-44.)

Everything else the kernels are particular about has a slower kernel behind it (head sizes
that are no multiple of 16, widths that are no multiple of 8, page sizes that are no power of
two run the plain 32-bit kernels), so it is no limit of the model.
"""

from __future__ import annotations

MAX_HEAD_DIM = 256  # the attention kernels keep a head's dims in the registers of one wavefront


def check_attention_sizes(num_heads: int, num_kv_heads: int, head_dim: int) -> None:
    """Raises ValueError for attention shapes no kernel of the library runs."""
    if head_dim > MAX_HEAD_DIM:
        raise ValueError(
            f"head_dim {head_dim}: the attention kernels take head sizes up to {MAX_HEAD_DIM} "
            f"({num_heads} query heads, {num_kv_heads} key/value heads asked for)"
        )
