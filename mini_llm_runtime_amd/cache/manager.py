"""The cache manager: pages of keys and values with a block table per request,
one pool per group of execution sites with equal needs, and fixed-size state
slots per request.

It is the single owner of page ids, block tables and slots, as the reference's
`PagedKVCacheManager` is of its allocator, storage and request registry
(src/mini_llm_runtime/paged_kv_manager.py:53-211).  The transaction rules are the
reference's (src/mini_llm_runtime/paged_kv_cache.py:202-243): a step begins by
taking the pages its tokens need (all requests or none), the model writes into
them, commit makes the tokens count, abort gives back only the pages this step
took and leaves the written bytes as invisible garbage.

Beyond the reference: several groups (each with pages and a free list of its
own), windows (pages that every later query has passed are given back at
commit), capacity promised by count instead of by pinning pages, and state slots.

What lives in a page, and in which order, is the business of the sites' cache specs
(`cache/spec.py`): the manager counts pages, rows and tokens and never asks what kind a
spec is.  A spec attaches its site to one of the two stores (`add_paged_site`,
`add_slot_site`), brings the tensors, and makes the view a mixer is handed.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Sequence, Union

import numpy as np
import torch

from .block_pool import BlockAllocator, BlockPoolExhaustedError, SlotPool, blocks_for
from .spec import PagedSpec, SiteCacheSpec, SlotSpec

SiteSpec = Optional[SiteCacheSpec]


class KVGroup:
    """Execution sites whose paged caches have equal specs share one pool: the tensors the spec
    makes (each [sites, pages, ...]) and one free list."""

    def __init__(
        self,
        index: int,
        spec: PagedSpec,
        sites: Sequence[int],
        num_blocks: int,
        block_size: int,
        dtype: torch.dtype,
        device: torch.device,
    ) -> None:
        self.index = index
        self.spec = spec
        self.sites = tuple(sites)
        self.site_position = {site: i for i, site in enumerate(self.sites)}
        self.allocator = BlockAllocator(num_blocks)
        self.block_size = block_size
        self.tensors: dict[str, torch.Tensor] = dict(spec.page_tensors(len(self.sites), num_blocks, block_size, dtype, device))
        for name, t in self.tensors.items():
            if t.dim() < 2 or tuple(t.shape[:2]) != (len(self.sites), num_blocks):
                raise ValueError(f"pool tensor {name!r} must be [sites, pages, ...], got {tuple(t.shape)}")

    @property
    def key(self) -> Optional[torch.Tensor]:
        return self.tensors.get("key")

    @property
    def value(self) -> Optional[torch.Tensor]:
        return self.tensors.get("value")

    def pages_of(self, site: int) -> dict[str, torch.Tensor]:
        """One site's share of the pool's tensors, each [pages, ...]."""
        i = self.site_position[site]
        return {name: t[i] for name, t in self.tensors.items()}

    @property
    def num_blocks(self) -> int:
        return self.allocator.total_blocks

    def dead_blocks(self, num_tokens: int) -> int:
        """How many leading pages no query at position >= num_tokens can see."""
        if self.spec.window is None:
            return 0
        first_visible = num_tokens - self.spec.window + 1
        return max(0, first_visible // self.block_size)

    def lifetime_blocks(self, max_tokens: int, max_step_tokens: int) -> int:
        """Most pages a request holds at one time over its life."""
        full = blocks_for(max_tokens, self.block_size)
        if self.spec.window is None:
            return full
        # the window before the first query of a step, the step's own tokens, and
        # one page for the misalignment of the window's start
        bounded = blocks_for(self.spec.window - 1 + max_step_tokens, self.block_size) + 1
        return min(full, bounded)

    def storage_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.tensors.values())


class StateBank:
    """Two copies of a fixed-size state per request slot: a step reads one and
    writes the other, commit swaps them, so an aborted step changes nothing.  Two spare rows
    behind them belong to nobody: the padded entries of a recorded step read and write those."""

    def __init__(self, site: int, spec: SlotSpec, num_slots: int, device: torch.device) -> None:
        self.site = site
        self.spec = spec
        self.tensor = spec.bank(num_slots * 2 + 2, device)
        if self.tensor.shape[0] != num_slots * 2 + 2:
            raise ValueError("a state bank must have two rows per request slot and two spare ones")


@dataclass
class RequestCache:
    request_id: str
    slot: int
    num_tokens: int = 0
    tables: list[list[int]] = field(default_factory=list)
    reserved: list[int] = field(default_factory=list)
    has_reservation: bool = False
    state_parity: int = 0
    pending_tokens: int = 0
    # `tables` as int32 arrays, per group (array, entries that are valid, `table_stamp` they were made at)
    table_arrays: dict = field(default_factory=dict, repr=False, compare=False)
    table_stamp: int = 0  # counts changes of `tables` other than appended pages

    def live_blocks(self, group: int) -> list[int]:
        return [b for b in self.tables[group] if b >= 0]

    def table_array(self, group: int) -> np.ndarray:
        """`tables[group]` as int32; kept between steps and only extended when pages were
        appended, rebuilt when the table changed in any other way."""
        table = self.tables[group]
        kept = self.table_arrays.get(group)
        n = len(table)
        if kept is not None:
            array, length, stamp = kept
            if stamp == self.table_stamp and length <= n:
                if length < n:
                    if n > array.shape[0]:
                        grown = np.empty(max(n, 2 * array.shape[0]), dtype=np.int32)
                        grown[:length] = array[:length]
                        array = grown
                    array[length:n] = table[length:]
                    self.table_arrays[group] = (array, n, stamp)
                return array[:n]
        array = np.empty(max(16, 2 * n), dtype=np.int32)
        array[:n] = table
        self.table_arrays[group] = (array, n, self.table_stamp)
        return array[:n]

    def tables_changed(self) -> None:
        """Entries of `tables` were overwritten or removed (not just appended)."""
        self.table_stamp += 1


@dataclass
class _PendingEntry:
    request: RequestCache
    num_new: int
    new_blocks: list[list[int]]
    from_reserved: list[int]


@dataclass
class StepLayout:
    """Host-side description of one step's tokens and where their cache lives."""

    request_ids: tuple[str, ...]
    q_starts: np.ndarray  # [R] tokens already cached
    q_lens: np.ndarray  # [R] tokens of this step
    context_lens: np.ndarray  # [R] q_start + q_len
    cu_q: np.ndarray  # [R+1]
    positions: np.ndarray  # [T]
    token_entry: np.ndarray  # [T] entry index of each token
    block_tables: list[np.ndarray]  # per group [R, max pages], -1 where no page
    slot_mappings: list[np.ndarray]  # per group [T] page * block_size + offset
    state_read: np.ndarray  # [R] row of the state banks to read
    state_write: np.ndarray  # [R] row to write
    slots: np.ndarray  # [R] request slot

    @property
    def num_tokens(self) -> int:
        return int(self.cu_q[-1])

    @property
    def num_entries(self) -> int:
        return len(self.request_ids)


@dataclass(frozen=True)
class CacheStats:
    """Counts as in the reference's `PagedCacheStats`
    (src/mini_llm_runtime/paged_kv_manager.py:34-50), per group."""

    group: int
    total_blocks: int
    free_blocks: int
    held_blocks: int
    reserved_blocks: int
    block_size: int
    allocated_slots: int
    committed_tokens: int
    pending_tokens: int
    internal_fragmentation_slots: int
    utilization: float
    storage_bytes: int


class VisibilityError(RuntimeError):
    """A site read the step's pending tokens before they were written, or a step was
    committed although a site that owns pages never wrote."""


class CacheManager:
    def __init__(
        self,
        site_specs: Sequence[SiteSpec],
        *,
        block_size: int,
        num_blocks: Union[int, Sequence[int]],
        max_requests: int,
        dtype: torch.dtype,
        device: Union[str, torch.device] = "cuda",
        check_visibility: bool = False,
    ) -> None:
        if block_size <= 0:
            raise ValueError("block_size must be > 0")
        if max_requests <= 0:
            raise ValueError("max_requests must be > 0")
        self.block_size = int(block_size)
        self.max_requests = int(max_requests)
        self.dtype = dtype
        self.device = torch.device(device)
        self.site_specs = tuple(site_specs)

        # every spec attaches its site to one of the two stores
        self._paged_sites: dict[PagedSpec, list[int]] = {}
        self.state_banks: dict[int, StateBank] = {}
        for site, spec in enumerate(self.site_specs):
            if spec is not None:
                spec.attach(self, site)
        grouped = self._paged_sites
        counts = [num_blocks] * len(grouped) if isinstance(num_blocks, int) else list(num_blocks)
        if len(counts) != len(grouped):
            raise ValueError(f"num_blocks names {len(counts)} pools, the model has {len(grouped)} groups")
        self.groups: list[KVGroup] = [
            KVGroup(i, spec, sites, int(counts[i]), self.block_size, dtype, self.device)
            for i, (spec, sites) in enumerate(grouped.items())
        ]
        self._site_group: dict[int, KVGroup] = {s: g for g in self.groups for s in g.sites}
        self.slots = SlotPool(self.max_requests)
        self._requests: dict[str, RequestCache] = {}
        self._pending: Optional[list[_PendingEntry]] = None
        # Debug check of what the reference's adapter enforces per layer
        # (src/mini_llm_runtime/paged_kv_adapter.py:109-147, 168-178): pending tokens of a site
        # may be read only after that site wrote them, and a step commits only when every
        # site that owns pages has written.  Mixers report through `KVView.written()` /
        # `KVView.reading()`; without the flag the reports cost nothing.
        self.check_visibility = bool(check_visibility)
        self._written_sites: set[int] = set()

    # ---- lookups ----------------------------------------------------------------
    @property
    def request_ids(self) -> tuple[str, ...]:
        return tuple(self._requests)

    def has_request(self, request_id: str) -> bool:
        return request_id in self._requests

    def get_request(self, request_id: str) -> RequestCache:
        try:
            return self._requests[request_id]
        except KeyError:
            raise KeyError(f"unknown request {request_id!r}") from None

    # ---- what the specs call -------------------------------------------------------------------
    def add_paged_site(self, site: int, spec: PagedSpec) -> None:
        """`site` keeps something per token in pages; sites with equal specs share a pool."""
        self._paged_sites.setdefault(spec, []).append(site)

    def add_slot_site(self, site: int, spec: SlotSpec) -> None:
        """`site` keeps a state of fixed size per request."""
        self.state_banks[site] = StateBank(site, spec, self.max_requests, self.device)

    def group_of_site(self, site: int) -> KVGroup:
        return self._site_group[site]

    def site_pools(self, site: int) -> tuple[torch.Tensor, torch.Tensor, int]:
        """(key pages, value pages, group index) of one site with keys and values in pages."""
        group = self._site_group[site]
        pages = group.pages_of(site)
        return pages["key"], pages["value"], group.index

    def site_view(self, site: int, owner: int, block_tables, slot_mappings, state_read, state_write):
        """What the mixer at execution site `site` is handed of the cache that site `owner` keeps
        (its own, or an earlier site's that it only reads), for a step whose metadata is given per
        pool (block tables, slot mappings) and per entry (state rows); None when `owner` keeps nothing.
        The view is made by the owner's spec."""
        group = self._site_group.get(owner)
        if group is not None:
            return group.spec.view(
                group.pages_of(owner),
                block_table=block_tables[group.index],
                slot_mapping=slot_mappings[group.index],
                block_size=self.block_size,
                writable=site == owner,
                site=site,
                owner=owner,
                tracker=self.visibility_tracker,
            )
        bank = self.state_banks.get(owner)
        if bank is not None:
            return bank.spec.view(bank.tensor, state_read, state_write)
        return None

    @property
    def step_in_flight(self) -> bool:
        return self._pending is not None

    @property
    def state_spare_rows(self) -> tuple[int, int]:
        """(row to read, row to write) of every state bank that no request owns."""
        return 2 * self.max_requests, 2 * self.max_requests + 1

    # ---- visibility of pending tokens (debug) ------------------------------------------------
    @property
    def visibility_tracker(self) -> Optional["CacheManager"]:
        """What a `KVView` reports to: this manager when the check is on, else None."""
        return self if self.check_visibility else None

    def note_write(self, site: int, owner: int) -> None:
        if self._pending is None:
            raise VisibilityError(f"site {site} wrote keys and values outside a step")
        if site != owner:
            raise VisibilityError(f"site {site} wrote into the pages of site {owner}, which it only reads")
        self._written_sites.add(owner)

    def note_read(self, site: int, owner: int) -> None:
        if self._pending is None:
            raise VisibilityError(f"site {site} read the cache outside a step")
        if owner not in self._written_sites:
            raise VisibilityError(
                f"site {site} reads the step's pending tokens of site {owner} before they were written"
            )

    def _unwritten_sites(self) -> list[int]:
        return [s for g in self.groups for s in g.sites if s not in self._written_sites]

    # ---- request lifetime ---------------------------------------------------------
    def create_request(self, request_id: str) -> RequestCache:
        if not request_id:
            raise ValueError("request_id must not be empty")
        if request_id in self._requests:
            raise ValueError(f"request {request_id!r} already exists")
        slot = self.slots.take()
        request = RequestCache(
            request_id=request_id,
            slot=slot,
            tables=[[] for _ in self.groups],
            reserved=[0 for _ in self.groups],
        )
        for bank in self.state_banks.values():
            bank.tensor[2 * slot : 2 * slot + 2].zero_()
        self._requests[request_id] = request
        return request

    def lifetime_blocks(self, max_tokens: int, max_step_tokens: int) -> list[int]:
        return [g.lifetime_blocks(max_tokens, max_step_tokens) for g in self.groups]

    def can_ever_hold(self, max_tokens: int, max_step_tokens: int) -> bool:
        need = self.lifetime_blocks(max_tokens, max_step_tokens)
        return all(n <= g.num_blocks for n, g in zip(need, self.groups))

    def try_create_reserved(self, request_id: str, max_tokens: int, max_step_tokens: int) -> bool:
        """Create a request and promise it the pages of its whole life, or do nothing.

        Returns False (no side effect) when a pool or the slots are short right now;
        raises ValueError when the request could never fit (as the reference's
        admission does, src/mini_llm_runtime/block_admission.py:43-49).
        """
        need = self.lifetime_blocks(max_tokens, max_step_tokens)
        for n, g in zip(need, self.groups):
            if n > g.num_blocks:
                raise ValueError(
                    f"request {request_id!r} can never be admitted: needs {n} pages of group {g.index}, "
                    f"the pool has {g.num_blocks}"
                )
        if self.slots.free_count == 0:
            return False
        if any(n > g.allocator.available_count for n, g in zip(need, self.groups)):
            return False
        request = self.create_request(request_id)
        for i, (n, g) in enumerate(zip(need, self.groups)):
            g.allocator.reserve(n)
            request.reserved[i] = n
        request.has_reservation = True
        return True

    def release_request(self, request_id: str) -> dict[int, tuple[int, ...]]:
        """Give back every page, promise and the slot; the request is gone afterwards."""
        request = self.get_request(request_id)
        if self._pending is not None and any(e.request is request for e in self._pending):
            raise RuntimeError(f"request {request_id!r} is part of the step in flight")
        released: dict[int, tuple[int, ...]] = {}
        for i, g in enumerate(self.groups):
            ids = request.live_blocks(i)
            g.allocator.free(ids)
            g.allocator.unreserve(request.reserved[i])
            released[i] = tuple(ids)
        self.slots.give_back(request.slot)
        del self._requests[request_id]
        return released

    # ---- one step = one transaction -------------------------------------------------
    def begin_step(self, entries: Sequence[tuple[str, int]]) -> StepLayout:
        """Take the pages the entries' new tokens need; all entries or none."""
        if self._pending is not None:
            raise RuntimeError("the previous step was neither committed nor aborted")
        if not entries:
            raise ValueError("a step needs at least one entry")
        seen: set[str] = set()
        for rid, n in entries:
            if rid in seen:
                raise ValueError(f"request {rid!r} appears twice in one step")
            seen.add(rid)
            if isinstance(n, bool) or not isinstance(n, (int, np.integer)) or n <= 0:
                raise ValueError(f"request {rid!r}: a step entry needs at least one token")
            self.get_request(rid)

        pending: list[_PendingEntry] = []
        try:
            for rid, n in entries:
                request = self._requests[rid]
                entry = _PendingEntry(request, int(n), [[] for _ in self.groups], [0 for _ in self.groups])
                pending.append(entry)
                for i, g in enumerate(self.groups):
                    have = len(request.tables[i])
                    need = blocks_for(request.num_tokens + int(n), self.block_size) - have
                    if need <= 0:
                        continue
                    promised = min(need, request.reserved[i])
                    ids = g.allocator.allocate(need, from_reserved=promised)
                    request.reserved[i] -= promised
                    request.tables[i].extend(ids)
                    entry.new_blocks[i] = ids
                    entry.from_reserved[i] = promised
        except BlockPoolExhaustedError:
            self._rollback(pending)
            raise
        for entry in pending:
            entry.request.pending_tokens = entry.num_new
        self._pending = pending
        self._written_sites.clear()
        return self._layout(pending)

    def _rollback(self, pending: list[_PendingEntry]) -> None:
        for entry in reversed(pending):
            request = entry.request
            for i, g in enumerate(self.groups):
                ids = entry.new_blocks[i]
                if not ids:
                    continue
                if request.tables[i][-len(ids) :] != ids:
                    raise RuntimeError("pages of an aborted step are no longer the table's tail")
                del request.tables[i][-len(ids) :]
                request.tables_changed()
                g.allocator.free(ids, to_reserved=entry.from_reserved[i])
                request.reserved[i] += entry.from_reserved[i]
            request.pending_tokens = 0

    def abort_step(self) -> None:
        if self._pending is None:
            raise RuntimeError("no step in flight")
        pending, self._pending = self._pending, None
        self._rollback(pending)

    def commit_step(self) -> dict[str, dict[int, tuple[int, ...]]]:
        """Make the step's tokens count; returns the window pages given back per request."""
        if self._pending is None:
            raise RuntimeError("no step in flight")
        if self.check_visibility:
            missing = self._unwritten_sites()
            if missing:
                raise VisibilityError(f"cannot commit: sites {missing} own pages and did not write this step's tokens")
        pending, self._pending = self._pending, None
        passed: dict[str, dict[int, tuple[int, ...]]] = {}
        for entry in pending:
            request = entry.request
            request.num_tokens += entry.num_new
            request.pending_tokens = 0
            request.state_parity ^= 1
            for i, g in enumerate(self.groups):
                dead = g.dead_blocks(request.num_tokens)
                ids = [b for b in request.tables[i][:dead] if b >= 0]
                if not ids:
                    continue
                keep = len(ids) if request.has_reservation else 0
                g.allocator.free(ids, to_reserved=keep)
                request.reserved[i] += keep
                for j in range(dead):
                    request.tables[i][j] = -1
                request.tables_changed()
                passed.setdefault(request.request_id, {})[i] = tuple(ids)
        return passed

    def _layout(self, pending: list[_PendingEntry]) -> StepLayout:
        bs = self.block_size
        count = len(pending)
        q_starts = np.array([e.request.num_tokens for e in pending], dtype=np.int32)
        q_lens = np.array([e.num_new for e in pending], dtype=np.int32)
        context = q_starts + q_lens
        cu_q = np.zeros(count + 1, dtype=np.int32)
        np.cumsum(q_lens, out=cu_q[1:])
        total = int(cu_q[-1])
        if total == count:  # one token each
            positions = q_starts.copy()
            token_entry = np.arange(count, dtype=np.int32)
        else:
            positions = np.empty(total, dtype=np.int32)
            token_entry = np.empty(total, dtype=np.int32)
            for r in range(count):
                a, b = int(cu_q[r]), int(cu_q[r + 1])
                positions[a:b] = np.arange(q_starts[r], context[r], dtype=np.int32)
                token_entry[a:b] = r
        used = (context + (bs - 1)) // bs  # pages each entry has with this step's tokens
        width = max(1, int(used.max()))
        block_tables: list[np.ndarray] = []
        slot_mappings: list[np.ndarray] = []
        for i, g in enumerate(self.groups):
            table = np.full((count, width), -1, dtype=np.int32)
            for r, e in enumerate(pending):
                n = int(used[r])
                table[r, :n] = e.request.table_array(i)[:n]
            pages = table[token_entry, positions // bs]
            if (pages < 0).any():
                r = int(token_entry[int(np.argmax(pages < 0))])
                raise RuntimeError(f"request {pending[r].request.request_id!r}: a new token has no page")
            block_tables.append(table)
            slot_mappings.append((pages * bs + positions % bs).astype(np.int32))
        slot_ids = np.array([e.request.slot for e in pending], dtype=np.int32)
        parity = np.array([e.request.state_parity for e in pending], dtype=np.int32)
        return StepLayout(
            request_ids=tuple(e.request.request_id for e in pending),
            q_starts=q_starts,
            q_lens=q_lens,
            context_lens=context.astype(np.int32),
            cu_q=cu_q,
            positions=positions,
            token_entry=token_entry,
            block_tables=block_tables,
            slot_mappings=slot_mappings,
            state_read=slot_ids * 2 + parity,
            state_write=slot_ids * 2 + (1 - parity),
            slots=slot_ids,
        )

    # ---- bookkeeping ------------------------------------------------------------------
    def stats(self) -> tuple[CacheStats, ...]:
        out = []
        for i, g in enumerate(self.groups):
            held = g.allocator.held_count
            committed = 0
            pending = 0
            for request in self._requests.values():
                live = len(request.live_blocks(i))
                dead_tokens = (len(request.tables[i]) - live) * self.block_size
                committed += max(0, request.num_tokens - dead_tokens)
                pending += request.pending_tokens
            allocated = held * self.block_size
            out.append(
                CacheStats(
                    group=i,
                    total_blocks=g.num_blocks,
                    free_blocks=g.allocator.free_count,
                    held_blocks=held,
                    reserved_blocks=g.allocator.reserved_count,
                    block_size=self.block_size,
                    allocated_slots=allocated,
                    committed_tokens=committed,
                    pending_tokens=pending,
                    internal_fragmentation_slots=allocated - committed - pending,
                    utilization=(committed / allocated) if allocated else 0.0,
                    storage_bytes=g.storage_bytes(),
                )
            )
        return tuple(out)

    def check_invariants(self) -> None:
        """No page lost, held twice or held by nobody; promises add up.  For tests and debugging."""
        for i, g in enumerate(self.groups):
            owned: list[int] = []
            promised = 0
            for request in self._requests.values():
                owned.extend(request.live_blocks(i))
                promised += request.reserved[i]
            if len(owned) != len(set(owned)):
                raise AssertionError(f"group {i}: a page is held by two tables")
            if sorted(owned) != g.allocator.held_ids():
                raise AssertionError(f"group {i}: the tables and the allocator disagree on held pages")
            if g.allocator.free_count + len(owned) != g.num_blocks:
                raise AssertionError(f"group {i}: pages were lost")
            if promised != g.allocator.reserved_count:
                raise AssertionError(f"group {i}: promised pages do not add up")
        slots = [r.slot for r in self._requests.values()]
        if len(slots) != len(set(slots)) or self.slots.free_count + len(slots) != self.max_requests:
            raise AssertionError("request slots are inconsistent")

    def poison(self) -> None:
        """Fill every page with NaN so that a read of an unwritten slot shows (tests)."""
        for g in self.groups:
            for t in g.tensors.values():
                if t.is_floating_point():
                    t.fill_(float("nan"))
