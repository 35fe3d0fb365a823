"""Knobs of the kernel library's launch heuristics.  Tests and measurements change them
through `HipOps(..., tuning=...)`; the defaults are what the measurements chose."""

from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class KernelTuning:
    decode_partition: int = 256  # keys per split of the decode attention
    decode_max_groups: int = 1024  # cap on the decode attention's workgroups
    max_k_slices: int = 16  # most partial sums a narrow product may be cut into
    fuse_norm: bool = True  # norm (+ residual) as the prologue of the product behind it, for few tokens
    fuse_merge: bool = True  # merge of the decode attention's splits as the prologue of the output product
    # A fused prologue is repeated by every workgroup of the product, and a compute unit takes in
    # only some 15 GB/s whatever the source: beyond this many bytes of prologue input per workgroup
    # the kernel of its own is the faster way.
    fuse_bytes: int = 1 << 30
    # The fused kernels stream weights in blocks of 16 rows, half as fast as the LDS-tiled kernel once a
    # matrix has tens of megabytes: beyond this many bytes of weight the norm and the merge keep kernels
    # of their own.  Decode steps at batch 1 with everything fused / with this limit: 1.5B (gate-up
    # 55 MB) 1.66 / 1.50 ms, 3B (90 MB) 2.42 / 2.25 ms, 7B (query/key/value 33 MB, output 26 MB)
    # 3.29 / 3.21 ms; the 17 MB gate-up of 0.5B stays fused (0.75 ms against 0.79).
    fuse_weight_bytes: int = 20 << 20
    # Prompt attention takes tiles of 128 queries instead of 64 once tiles x heads reach this many
    # workgroups (fewer leave compute units idle behind the heaviest tiles).
    # Behind thousands of cached keys every tile is heavy and three quarters of that are enough.
    wide_attention_groups: int = 512
    # Behind twice as many keys, fewer workgroups than this have the keys of every tile cut into
    # runs (up to 8) with a workgroup each, until there are this many.
    key_run_groups: int = 384

    # The last product of a part (output projection, down projection) as a kernel that owns whole
    # output columns and adds them to the residual stream itself, with the next norm left as one
    # factor per row for the product behind it: one kernel instead of a product cut along k plus a
    # norm kernel.  Measured inside a replayed graph at 0.5B sizes (microseconds a call, weights of 24
    # layers in turn): the norm kernel it saves costs 2.7, the product that owns its columns costs 1.0
    # more than the one cut along k for the output projection (1.6 MB: 4.4 against 3.3) and 3.0 more
    # for the down projection (8.7 MB, k = 4,864: 7.9 against 4.9: few workgroups, each held to the
    # 20 GB/s that a compute unit takes in), and the consumer's scaling costs 0.7 to 1.0.  So it pays
    # for small matrices only, 0.7 us a layer at 5 to 8 tokens, and loses everywhere else: below 5
    # tokens to the norm done in the consumer's prologue, from 9 tokens on to the activations that
    # every workgroup reads.  The limits below say where it is used.
    finish_stream: bool = True
    finish_weight_bytes: int = 4 << 20
    finish_activation_bytes: int = 160 << 10
    finish_min_tokens: int = 5
    finish_max_tokens: int = 8
    # (For more than 64 tokens the same was tried as an epilogue of the tiled kernels and lost: 0.5B
    # prompt of 2,048 tokens 4.31 to 4.47 ms.  A lane of the matrix cores' accumulator holds four
    # features of ONE token, so the float32 stream is read and written 16 bytes at a time at a stride of
    # a row, where the norm kernel reads whole rows.)

    def __post_init__(self) -> None:
        for name in ("decode_partition", "decode_max_groups", "max_k_slices", "wide_attention_groups", "key_run_groups", "fuse_weight_bytes",
                     "finish_weight_bytes", "finish_activation_bytes", "finish_min_tokens",
                     "finish_max_tokens"):
            value = getattr(self, name)
            if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
                raise ValueError(f"KernelTuning.{name} must be a positive integer")
