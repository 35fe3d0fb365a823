"""Admission by pages: a request enters only when the pages of its whole life can
be promised to it, so that no running request ever runs out of pages.

Behaviour of the reference's `PagedBlockAdmissionController`
(src/mini_llm_runtime/block_admission.py:18-93): `try_admit` either creates the
request in the cache manager with its capacity set aside, or changes nothing and
returns False; a request that could never fit raises; finished (or un-admitted)
requests give everything back.  The promise here is a count per page pool, not a
set of pinned pages.
"""

from __future__ import annotations

from dataclasses import dataclass

from ..cache.manager import CacheManager
from .scheduler import RequestState


@dataclass(frozen=True)
class BlockReservation:
    request_id: str
    max_cache_tokens: int
    block_counts: tuple[int, ...]  # per page pool


class PagedBlockAdmissionController:
    def __init__(self, manager: CacheManager, *, max_step_tokens: int) -> None:
        if max_step_tokens <= 0:
            raise ValueError("max_step_tokens must be > 0")
        self.manager = manager
        self.max_step_tokens = int(max_step_tokens)
        self._reservations: dict[str, BlockReservation] = {}

    @property
    def reservations(self) -> tuple[BlockReservation, ...]:
        return tuple(self._reservations.values())

    def reservation_for(self, request_id: str) -> BlockReservation:
        try:
            return self._reservations[request_id]
        except KeyError:
            raise KeyError(f"request {request_id!r} has no reservation") from None

    def try_admit(self, request: RequestState) -> bool:
        if request.request_id in self._reservations:
            raise RuntimeError(f"request {request.request_id!r} is already admitted")
        tokens = request.max_cache_tokens
        if not self.manager.try_create_reserved(request.request_id, tokens, self.max_step_tokens):
            return False
        self._reservations[request.request_id] = BlockReservation(
            request_id=request.request_id,
            max_cache_tokens=tokens,
            block_counts=tuple(self.manager.lifetime_blocks(tokens, self.max_step_tokens)),
        )
        return True

    def release_finished(self, request_ids: tuple[str, ...]) -> dict[str, dict[int, tuple[int, ...]]]:
        return self.release_admitted(request_ids)

    def release_admitted(self, request_ids: tuple[str, ...]) -> dict[str, dict[int, tuple[int, ...]]]:
        """Give back the pages and promises of admitted requests (finished, or un-admitted after a failed step)."""
        if len(set(request_ids)) != len(request_ids):
            raise ValueError("request ids must not repeat")
        missing = [rid for rid in request_ids if rid not in self._reservations]
        if missing:
            raise KeyError(f"requests without a reservation: {missing}")
        released = {}
        for rid in request_ids:
            released[rid] = self.manager.release_request(rid)
            del self._reservations[rid]
        return released
