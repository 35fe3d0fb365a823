"""What the attention kernels want to know about a batch before they are launched: the plan
a mixer that uses them hands to the step function, which uploads its arrays with the step's
other metadata and makes its sizes part of a recorded step's identity.
"""

from __future__ import annotations

import numpy as np

from ..parts.context import MixerPlan, PlanInput

QUERY_TILE = 64  # queries of one request that the prompt kernel takes together
WIDE_QUERY_TILE = 128  # and in its variant for long prompts (two blocks of queries per wavefront)
LONG_PREFIX_KEYS = 2048  # mean number of keys before a tile from which a step counts as behind long prefixes (twice: very long)
PAGED_ATTENTION = "paged_attention"  # the plan's key: every mixer on these kernels shares one plan per step


def query_tiles(q_lens, q_starts=None, tile: int = QUERY_TILE) -> np.ndarray:
    """[num_tiles, 2] int32 (entry, first query) covering every entry with more than one new
    token in tiles of `tile` queries, the tiles with the most keys before them first: a kernel
    that hands them to the compute units in that order can start the heavy ones early and pair
    them with light ones."""
    tiles = [(r, q0) for r, n in enumerate(q_lens) if n > 1 for q0 in range(0, int(n), tile)]
    if q_starts is None:
        q_starts = [0] * len(q_lens)
    tiles.sort(key=lambda t: -(int(q_starts[t[0]]) + t[1]))
    return np.asarray(tiles, dtype=np.int32).reshape(-1, 2)


def attention_plan(shape: PlanInput) -> MixerPlan:
    """Tiles of 64 and of 128 queries over the entries with several new tokens (for the prompt
    kernel and its wide variant; the launch picks one by how many there are), and
    how many entries have a single token and how long their contexts may be (for the split-KV
    decode kernel).  `shape.max_context` bounds the contexts; a recording is made with the
    capacity of its block tables there, so that it holds for every later step of its sizes."""
    single = shape.q_lens == 1
    decodes = int(single.sum())
    tiles = query_tiles(shape.q_lens, shape.q_starts)
    wide = query_tiles(shape.q_lens, shape.q_starts, WIDE_QUERY_TILE)
    # portions behind long cached prefixes: every tile has thousands of keys before it, so fewer
    # tiles keep the compute units busy for long and the wide tiles' lower cost per key wins
    # (level 1); behind twice as many (level 2) few tiles have their keys cut into runs
    keys_before = [int(shape.q_starts[e]) + int(q0) for e, q0 in wide]
    mean_before = sum(keys_before) / len(keys_before) if keys_before else 0
    long_prefix = int(mean_before >= LONG_PREFIX_KEYS) + int(mean_before >= 2 * LONG_PREFIX_KEYS)
    return MixerPlan(
        key=PAGED_ATTENTION,
        arrays={"query_tiles": tiles, "wide_query_tiles": wide},
        sizes={
            "num_query_tiles": len(tiles),
            "num_wide_query_tiles": len(wide),
            "long_prefix": long_prefix,
            "num_decode_entries": decodes,
            "max_decode_context": int(shape.max_context) if decodes else 0,
        },
    )
