"""The cache manager on the CPU: page order, all-or-nothing calls, transactions,
reuse, windows, promises, slots; and under random orders of requests no page is
lost, held twice or freed twice."""

from __future__ import annotations

import random

import pytest
import torch

from mini_llm_runtime_amd.cache import (
    BlockAllocator,
    BlockPoolExhaustedError,
    CacheManager,
    PagedKVSpec,
    SlotStateSpec,
)


def make(num_blocks=8, block_size=4, specs=None, max_requests=4):
    specs = specs if specs is not None else [PagedKVSpec(2, 8), PagedKVSpec(2, 8)]
    return CacheManager(specs, block_size=block_size, num_blocks=num_blocks, max_requests=max_requests,
                        dtype=torch.float32, device="cpu")


# ---- allocator (reference tests/test_paged_kv_cache.py:11-60) -------------------------------------
def test_allocator_order_reuse_and_atomic_failures():
    a = BlockAllocator(4)
    assert a.allocate(2) == [0, 1]
    assert a.allocate(1) == [2]
    with pytest.raises(BlockPoolExhaustedError):
        a.allocate(2)
    assert a.free_count == 1  # the failed call changed nothing
    a.free([1])
    assert a.allocate(2) == [1, 3]  # lowest id first
    with pytest.raises(ValueError):
        a.free([0, 0])
    with pytest.raises(ValueError):
        a.free([0, 7])
    assert a.held_count == 4  # a refused free changed nothing
    a.free([0])
    with pytest.raises(ValueError, match="not held"):
        a.free([0])


def test_allocator_promises():
    a = BlockAllocator(4)
    a.reserve(3)
    assert a.available_count == 1
    with pytest.raises(BlockPoolExhaustedError):
        a.allocate(2)
    assert a.allocate(2, from_reserved=2) == [0, 1]
    assert (a.reserved_count, a.available_count) == (1, 1)
    with pytest.raises(BlockPoolExhaustedError):
        a.reserve(2)
    a.free([0], to_reserved=1)
    assert (a.reserved_count, a.free_count) == (2, 3)


# ---- tables and transactions (reference tests/test_paged_kv_cache.py:63-153) ----------------------------
def test_groups_layout_and_growth_across_pages():
    m = make()
    assert len(m.groups) == 1 and m.groups[0].sites == (0, 1)
    assert m.groups[0].key.shape == (2, 8, 2, 4, 8)
    m.create_request("a")
    lay = m.begin_step([("a", 5)])
    assert lay.positions.tolist() == [0, 1, 2, 3, 4]
    assert lay.block_tables[0].tolist() == [[0, 1]]
    assert lay.slot_mappings[0].tolist() == [0, 1, 2, 3, 4]
    assert m.get_request("a").num_tokens == 0  # pending tokens do not count before commit
    m.commit_step()
    assert m.get_request("a").num_tokens == 5
    lay = m.begin_step([("a", 4)])  # fills the partial page first, then takes one more
    assert lay.q_starts.tolist() == [5] and lay.context_lens.tolist() == [9]
    assert lay.block_tables[0].tolist() == [[0, 1, 2]]
    assert lay.slot_mappings[0].tolist() == [5, 6, 7, 8]
    m.commit_step()
    m.check_invariants()


def test_abort_returns_only_new_pages_and_nested_begin_is_refused():
    m = make()
    m.create_request("a")
    m.begin_step([("a", 3)])
    with pytest.raises(RuntimeError):
        m.begin_step([("a", 1)])
    m.commit_step()
    m.begin_step([("a", 6)])  # needs pages 1 and 2
    assert m.groups[0].allocator.free_count == 5
    m.abort_step()
    assert m.groups[0].allocator.free_count == 7
    assert m.get_request("a").tables[0] == [0] and m.get_request("a").num_tokens == 3
    with pytest.raises(RuntimeError):
        m.abort_step()
    m.check_invariants()


def test_step_is_all_or_nothing_across_requests():
    m = make(num_blocks=3)
    m.create_request("a")
    m.create_request("b")
    with pytest.raises(BlockPoolExhaustedError):
        m.begin_step([("a", 8), ("b", 5)])  # a takes 2 pages, b would need 2 more
    assert m.groups[0].allocator.free_count == 3
    assert m.get_request("a").tables[0] == [] and not m.step_in_flight
    m.check_invariants()


def test_release_and_reuse_and_unknown_requests():
    m = make(num_blocks=4)
    m.create_request("a")
    m.begin_step([("a", 7)])
    m.commit_step()
    m.create_request("b")
    m.begin_step([("b", 2)])
    with pytest.raises(RuntimeError):
        m.release_request("b")  # part of the step in flight
    m.commit_step()
    assert m.release_request("a") == {0: (0, 1)}
    with pytest.raises(KeyError):
        m.get_request("a")
    with pytest.raises(KeyError):
        m.begin_step([("a", 1)])
    m.create_request("c")
    lay = m.begin_step([("c", 5)])
    assert lay.block_tables[0].tolist() == [[0, 1]]  # freed pages are handed out again
    m.commit_step()
    with pytest.raises(ValueError):
        m.create_request("c")
    with pytest.raises(ValueError):
        m.begin_step([("b", 1), ("b", 1)])
    m.check_invariants()


def test_stats_identity():
    m = make(block_size=4)
    m.create_request("a")
    m.begin_step([("a", 6)])
    s = m.stats()[0]
    assert (s.held_blocks, s.allocated_slots, s.committed_tokens, s.pending_tokens) == (2, 8, 0, 6)
    assert s.allocated_slots - s.committed_tokens - s.pending_tokens == s.internal_fragmentation_slots == 2
    m.commit_step()
    s = m.stats()[0]
    assert (s.committed_tokens, s.pending_tokens, s.utilization) == (6, 0, 0.75)
    assert s.storage_bytes == 2 * 2 * 8 * 2 * 4 * 8 * 4


# ---- groups with different needs ---------------------------------------------------------------------
def test_window_group_gives_back_passed_pages():
    specs = [PagedKVSpec(2, 8), PagedKVSpec(2, 8, window=6), PagedKVSpec(2, 8)]
    m = make(num_blocks=[16, 4], block_size=4, specs=specs)
    assert [g.sites for g in m.groups] == [(0, 2), (1,)]
    m.create_request("a")
    m.begin_step([("a", 7)])
    m.commit_step()  # next query at 7 sees keys 2..7: page 0 (keys 0..3) is still needed
    assert m.get_request("a").tables[1] == [0, 1]
    lay = m.begin_step([("a", 3)])  # tokens 7, 8, 9
    assert lay.block_tables[1].tolist() == [[0, 1, 2]]
    passed = m.commit_step()  # next query at 10 sees keys 5..10: page 0 has passed
    assert passed == {"a": {1: (0,)}}
    assert m.get_request("a").tables[1] == [-1, 1, 2]
    assert m.get_request("a").tables[0] == [0, 1, 2]  # the full-attention group keeps everything
    for _ in range(30):  # a long decode never needs more than 3 pages of the window pool
        lay = m.begin_step([("a", 1)])
        m.commit_step()
        assert len(m.get_request("a").live_blocks(1)) <= 3
    assert lay.block_tables[1][0, 0] == -1
    m.check_invariants()
    m.release_request("a")
    assert all(g.allocator.free_count == g.num_blocks for g in m.groups)


def test_lifetime_promise_admission():
    m = make(num_blocks=5, block_size=4)
    assert m.try_create_reserved("a", 12, 8) is True  # 3 pages promised, none taken
    g = m.groups[0].allocator
    assert (g.free_count, g.reserved_count, g.available_count) == (5, 3, 2)
    assert m.try_create_reserved("b", 9, 8) is False  # needs 3, only 2 are not promised: no side effect
    assert not m.has_request("b") and g.reserved_count == 3
    with pytest.raises(ValueError, match="never"):
        m.try_create_reserved("c", 100, 8)
    assert m.try_create_reserved("b", 8, 8) is True
    m.begin_step([("a", 9), ("b", 4)])  # draws on the promises
    m.commit_step()
    assert (g.free_count, g.reserved_count) == (1, 1)
    m.create_request("x")  # an unpromised request cannot take a's last promised page
    with pytest.raises(BlockPoolExhaustedError):
        m.begin_step([("x", 1)])
    m.begin_step([("a", 3)])
    m.commit_step()
    m.check_invariants()
    m.release_request("a")
    m.release_request("b")
    m.release_request("x")
    assert (g.free_count, g.reserved_count) == (5, 0)


def test_state_slots_are_double_buffered():
    specs = [PagedKVSpec(1, 4), SlotStateSpec((3,))]
    m = make(specs=specs, max_requests=2)
    bank = m.state_banks[1].tensor
    assert bank.shape == (6, 3) and m.state_spare_rows == (4, 5)  # two rows per slot, two that nobody owns
    a = m.create_request("a")
    b = m.create_request("b")
    assert (a.slot, b.slot) == (0, 1)
    with pytest.raises(BlockPoolExhaustedError):
        m.create_request("c")
    lay = m.begin_step([("b", 2), ("a", 1)])
    assert lay.state_read.tolist() == [2, 0] and lay.state_write.tolist() == [3, 1]
    bank[3] = 5.0
    m.abort_step()  # an aborted step leaves the readable copy untouched
    lay = m.begin_step([("b", 2)])
    assert lay.state_read.tolist() == [2]
    m.commit_step()
    lay = m.begin_step([("b", 1)])
    assert lay.state_read.tolist() == [3] and lay.state_write.tolist() == [2]
    m.commit_step()
    m.release_request("a")
    c = m.create_request("c")
    assert c.slot == 0 and torch.equal(bank[0:2], torch.zeros(2, 3))  # zeroed at admission


# ---- random orders ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_every_page_accounted_for(seed):
    rng = random.Random(seed)
    specs = [PagedKVSpec(2, 8), PagedKVSpec(2, 8, window=rng.choice([5, 9, 17])), PagedKVSpec(1, 16)]
    m = make(num_blocks=[rng.randint(6, 14)] * 3, block_size=rng.choice([2, 4, 8]), specs=specs, max_requests=5)
    live: dict[str, int] = {}
    counter = 0
    for _ in range(400):
        action = rng.random()
        if action < 0.25 and len(live) < 5:
            rid = f"r{counter}"
            counter += 1
            if rng.random() < 0.5:
                try:
                    ok = m.try_create_reserved(rid, rng.randint(1, 40), 8)
                except ValueError:
                    ok = False
                if ok:
                    live[rid] = 0
            else:
                m.create_request(rid)
                live[rid] = 0
        elif action < 0.85 and live:
            chosen = rng.sample(sorted(live), rng.randint(1, len(live)))
            entries = [(rid, rng.randint(1, 8)) for rid in chosen]
            before = [g.allocator.free_count for g in m.groups]
            try:
                lay = m.begin_step(entries)
            except BlockPoolExhaustedError:
                assert [g.allocator.free_count for g in m.groups] == before
                m.check_invariants()
                continue
            for gi, g in enumerate(m.groups):  # every new token has a slot in a page the request holds
                slots = lay.slot_mappings[gi]
                assert len(set(slots.tolist())) == len(slots)
                for t, s in enumerate(slots):
                    rid = lay.request_ids[int(lay.token_entry[t])]
                    assert int(s) // m.block_size in m.get_request(rid).live_blocks(gi)
            if rng.random() < 0.2:
                m.abort_step()
                assert [g.allocator.free_count for g in m.groups] == before
            else:
                m.commit_step()
                for rid, n in entries:
                    live[rid] += n
                    assert m.get_request(rid).num_tokens == live[rid]
        elif live:
            rid = rng.choice(sorted(live))
            m.release_request(rid)
            del live[rid]
            with pytest.raises(KeyError):
                m.release_request(rid)
        m.check_invariants()
    for rid in list(live):
        m.release_request(rid)
    m.check_invariants()
    assert all(g.allocator.free_count == g.num_blocks and g.allocator.reserved_count == 0 for g in m.groups)
    assert m.slots.free_count == 5
