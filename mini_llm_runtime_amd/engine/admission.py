"""Admission by pages: a request enters only when the pages of its whole life can be
promised to it, so that no admitted request ever runs out of pages.

What the reference's admission controller decides (src/mini_llm_runtime/block_admission.py:18-93):
either the request is created in the cache manager with its capacity set aside, or nothing
changes and the answer is no; a request that could never fit is an error; a request that ends
(or is un-admitted after a failed step) gives everything back.  The promise here is a count per
page pool that the cache manager keeps, not a set of pinned pages.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Iterable

from ..cache.manager import CacheManager
from .request import Request


@dataclass(frozen=True)
class PagePromise:
    request_id: str
    tokens: int  # most tokens the request ever caches
    pages: tuple[int, ...]  # promised per page pool


class PageAdmission:
    def __init__(self, manager: CacheManager, *, max_step_tokens: int) -> None:
        if max_step_tokens <= 0:
            raise ValueError("max_step_tokens must be > 0")
        self.manager = manager
        self.max_step_tokens = int(max_step_tokens)
        self._promises: dict[str, PagePromise] = {}

    @property
    def promises(self) -> tuple[PagePromise, ...]:
        return tuple(self._promises.values())

    def pages_for(self, tokens: int) -> tuple[int, ...]:
        return tuple(self.manager.lifetime_blocks(tokens, self.max_step_tokens))

    def can_ever_admit(self, tokens: int) -> bool:
        """Whether empty pools could hold a request that caches this many tokens."""
        return self.manager.can_ever_hold(tokens, self.max_step_tokens)

    def admit(self, request: Request) -> bool:
        if request.id in self._promises:
            raise RuntimeError(f"request {request.id!r} is already admitted")
        if not self.manager.try_create_reserved(request.id, request.cache_tokens, self.max_step_tokens):
            return False
        self._promises[request.id] = PagePromise(request.id, request.cache_tokens, self.pages_for(request.cache_tokens))
        return True

    def release(self, request_ids: Iterable[str]) -> dict[str, dict[int, tuple[int, ...]]]:
        """Requests that ended, or were un-admitted, give back their pages, promises and slots;
        returns the pages each one held, per pool."""
        ids = tuple(request_ids)
        unknown = [rid for rid in ids if rid not in self._promises]
        if unknown or len(set(ids)) != len(ids):
            raise KeyError(f"not admitted, or named twice: {unknown or ids}")
        freed = {}
        for rid in ids:
            freed[rid] = self.manager.release_request(rid)
            del self._promises[rid]
        return freed
