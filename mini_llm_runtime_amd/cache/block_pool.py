"""Page ids of one pool: a free list on the host, all-or-nothing calls.

Behaviour follows the reference's `FixedBlockAllocator`
(src/mini_llm_runtime/paged_kv_cache.py:36-113): ids come out in the order
0, 1, 2, ...; freed ids are reused lowest first; a failed call changes nothing;
freeing an id that is not held is an error.  Added here: a count of pages that
are promised to admitted requests but not yet taken (`reserved`), so admission
can keep capacity for a request's lifetime without pinning physical pages.
"""

from __future__ import annotations

from typing import Iterable, Sequence


class BlockPoolExhaustedError(RuntimeError):
    """Not enough free pages; raised before any state is changed."""


class BlockAllocator:
    def __init__(self, total_blocks: int) -> None:
        if isinstance(total_blocks, bool) or not isinstance(total_blocks, int) or total_blocks <= 0:
            raise ValueError("total_blocks must be a positive integer")
        self.total_blocks = total_blocks
        # a stack whose top is the lowest id
        self._free: list[int] = list(range(total_blocks - 1, -1, -1))
        self._held = bytearray(total_blocks)
        self._reserved = 0

    # ---- counts -------------------------------------------------------------
    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def held_count(self) -> int:
        return self.total_blocks - len(self._free)

    @property
    def reserved_count(self) -> int:
        """Pages promised to admitted requests and not yet taken."""
        return self._reserved

    @property
    def available_count(self) -> int:
        """Free pages that are not promised to anyone."""
        return len(self._free) - self._reserved

    def is_held(self, block_id: int) -> bool:
        return 0 <= block_id < self.total_blocks and bool(self._held[block_id])

    # ---- reservations ---------------------------------------------------------
    def reserve(self, count: int) -> None:
        if count < 0:
            raise ValueError("count must be >= 0")
        if count > self.available_count:
            raise BlockPoolExhaustedError(
                f"cannot reserve {count} pages: {self.available_count} available of {self.total_blocks}"
            )
        self._reserved += count

    def unreserve(self, count: int) -> None:
        if count < 0 or count > self._reserved:
            raise ValueError(f"cannot give back {count} reserved pages, {self._reserved} are reserved")
        self._reserved -= count

    # ---- pages ----------------------------------------------------------------
    def allocate(self, count: int, *, from_reserved: int = 0) -> list[int]:
        """Take `count` pages; `from_reserved` of them were promised to the caller."""
        if count < 0 or from_reserved < 0 or from_reserved > count:
            raise ValueError("bad allocate() arguments")
        if from_reserved > self._reserved:
            raise ValueError("caller claims more reserved pages than are reserved")
        unpromised = count - from_reserved
        if unpromised > self.available_count:
            raise BlockPoolExhaustedError(
                f"need {count} pages ({from_reserved} reserved): "
                f"{self.available_count} available, {len(self._free)} free of {self.total_blocks}"
            )
        ids = [self._free.pop() for _ in range(count)]
        for i in ids:
            self._held[i] = 1
        self._reserved -= from_reserved
        return ids

    def free(self, block_ids: Iterable[int], *, to_reserved: int = 0) -> None:
        """Give pages back; `to_reserved` of them stay promised to the caller."""
        ids = list(block_ids)
        if to_reserved < 0 or to_reserved > len(ids):
            raise ValueError("bad free() arguments")
        seen: set[int] = set()
        for i in ids:
            if isinstance(i, bool) or not isinstance(i, int) or not 0 <= i < self.total_blocks:
                raise ValueError(f"page id {i!r} is outside the pool")
            if not self._held[i] or i in seen:
                raise ValueError(f"page {i} is not held (freed twice?)")
            seen.add(i)
        for i in ids:
            self._held[i] = 0
        # lowest id on top, so it is the next one handed out
        self._free.extend(sorted(ids, reverse=True))
        self._free.sort(reverse=True)
        self._reserved += to_reserved

    def held_ids(self) -> list[int]:
        return [i for i in range(self.total_blocks) if self._held[i]]


class SlotPool:
    """Indices of fixed-size per-request state slots."""

    def __init__(self, num_slots: int) -> None:
        if num_slots <= 0:
            raise ValueError("num_slots must be > 0")
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))
        self._held = bytearray(num_slots)

    @property
    def free_count(self) -> int:
        return len(self._free)

    def take(self) -> int:
        if not self._free:
            raise BlockPoolExhaustedError("no free request slot")
        slot = self._free.pop()
        self._held[slot] = 1
        return slot

    def give_back(self, slot: int) -> None:
        if not 0 <= slot < self.num_slots or not self._held[slot]:
            raise ValueError(f"slot {slot} is not held")
        self._held[slot] = 0
        self._free.append(slot)
        self._free.sort(reverse=True)


def ceil_div(a: int, b: int) -> int:
    return -(-a // b)


def blocks_for(tokens: int, block_size: int) -> int:
    return ceil_div(tokens, block_size) if tokens > 0 else 0


__all__: Sequence[str] = (
    "BlockAllocator",
    "BlockPoolExhaustedError",
    "SlotPool",
    "blocks_for",
    "ceil_div",
)
