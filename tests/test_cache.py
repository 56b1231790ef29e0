"""The cache's bookkeeping: no slot or page is lost, held twice or freed twice; a step reserves
everything or nothing; groups with different needs have storage of their own."""

import random

import pytest
import torch

from beholdd.cache import CacheError, CacheFull, SequenceCache
from beholdd.parts import CacheNeed

KV = CacheNeed(kind="kv", kv_heads=2, head_dim=16)
WINDOWED = CacheNeed(kind="kv", kv_heads=2, head_dim=16, window=100)
STATE = CacheNeed(kind="state", state_shape=(3, 5), state_dtype=torch.float32)


def make(needs=None, max_tokens=640, **kw):
    cache = SequenceCache(needs or {0: KV, 1: KV}, max_tokens, torch.float32, "cpu", 64, **kw)
    cache.allocate()
    return cache


def test_sizes_follow_max_tokens_in_pages_of_64():
    assert make(max_tokens=640).n_pages == 10 and make(max_tokens=641).n_pages == 11 and make(max_tokens=1).n_pages == 1
    cache = make(max_tokens=640)
    assert cache.groups[0].k.shape == (2, 10, 2, 64, 16) and cache.groups[0].v.shape == (2, 10, 2, 16, 64)


def test_byte_accounting_equals_what_is_allocated():
    needs = {0: KV, 1: KV, 2: WINDOWED, 3: STATE, 4: STATE}
    cache = SequenceCache(needs, 1000, torch.bfloat16, "cpu", 64, max_slots=7)
    plan = cache.plan()
    assert cache.allocated_bytes() == 0                     # the plan is made before anything is allocated
    cache.allocate()
    assert plan.total_bytes == cache.allocated_bytes()
    assert len(cache.groups) == 3                           # full keys, windowed keys and state: storage of their own
    kinds = sorted((g.need.kind, g.need.window, len(g.entries)) for g in cache.groups)
    assert kinds == [("kv", 0, 2), ("kv", 100, 1), ("state", 0, 2)]
    assert "16 pages of 64 tokens" in plan.describe()
    with pytest.raises(CacheFull, match="limit"):
        SequenceCache(needs, 1000, torch.bfloat16, "cpu", 64).allocate(limit_bytes=1000)


def test_slots_are_given_back_and_used_again():
    cache = make(max_slots=3)
    a, b, c = cache.alloc_slot(), cache.alloc_slot(), cache.alloc_slot()
    assert (a, b, c) == (0, 1, 2)
    with pytest.raises(CacheFull, match="slots"):
        cache.alloc_slot()
    cache.free_slot(b)
    assert cache.alloc_slot() == b                          # used again at once
    cache.free_slot(a)
    with pytest.raises(CacheError, match="not in use"):
        cache.free_slot(a)                                  # freed twice
    with pytest.raises(CacheError, match="not in use"):
        cache.free_slot(99)
    with pytest.raises(CacheError, match="not in use"):
        cache.length(a)
    cache.check_invariants()


def test_reserve_takes_everything_or_nothing():
    cache = make(max_tokens=256)                            # four pages
    a, b = cache.alloc_slot(), cache.alloc_slot()
    cache.reserve([(a, 100), (b, 64)])                      # 2 + 1 pages
    cache.commit([(a, 100), (b, 64)])
    assert cache.length(a) == 100 and cache.length(b) == 64 and cache.free_page_count() == 1
    with pytest.raises(CacheFull, match="pages"):
        cache.reserve([(a, 29), (b, 1)])                    # a needs a third page, b a second: only one is free
    assert cache.free_page_count() == 1 and cache.length(a) == 100
    cache.check_invariants()
    cache.reserve([(a, 28), (b, 1)])                        # a still fits its second page
    cache.rollback([(a, 28), (b, 1)])                       # the step failed: b's new page goes back
    assert cache.free_page_count() == 1
    with pytest.raises(CacheError, match="twice"):
        cache.reserve([(a, 1), (a, 1)])
    with pytest.raises(CacheError, match="at least one token"):
        cache.reserve([(a, 0)])
    cache.free_slot(a)
    assert cache.free_page_count() == 3
    cache.check_invariants()


def test_positions_are_bounded_by_the_model(): 
    cache = make(max_tokens=640, max_position=128)
    slot = cache.alloc_slot()
    cache.reserve([(slot, 128)])
    cache.commit([(slot, 128)])
    with pytest.raises(CacheFull, match="exceed the limit of 128"):
        cache.reserve([(slot, 1)])


def test_page_tables_follow_positions():
    cache = make(max_tokens=640)
    a, b = cache.alloc_slot(), cache.alloc_slot()
    cache.reserve([(a, 65), (b, 1)])
    cache.commit([(a, 65), (b, 1)])
    tables = cache.page_tables([b, a])
    table = tables[0]
    assert table.dtype == torch.int32 and table.shape == (2, 2)
    pages_a, pages_b = cache.groups[0].pages_of[a], cache.groups[0].pages_of[b]
    assert table[1].tolist() == pages_a and table[0].tolist() == pages_b + [0]
    assert len(set(pages_a + pages_b)) == 3
    layer = cache.layer_cache(1, True, tables)
    assert layer.k_pages.data_ptr() == cache.groups[0].k[1].data_ptr() and layer.page_table is table


def test_a_window_gives_pages_back_as_the_sequence_moves_on():
    cache = make({0: KV, 1: WINDOWED}, max_tokens=1024)
    full = [g for g in cache.groups if not g.need.window][0]
    windowed = [g for g in cache.groups if g.need.window][0]
    slot = cache.alloc_slot()
    cache.reserve([(slot, 300)])
    cache.commit([(slot, 300)])
    # the next query stands at 300 and sees 201..300: pages 0, 1 and 2 (positions 0..191) are dead
    assert windowed.pages_of[slot][:3] == [-1, -1, -1] and windowed.pages_of[slot][3] >= 0
    assert all(p >= 0 for p in full.pages_of[slot])
    assert len(windowed.free_pages) == 16 - 2 and len(full.free_pages) == 16 - 5
    cache.check_invariants()
    cache.free_slot(slot)
    assert len(windowed.free_pages) == 16 and len(full.free_pages) == 16
    cache.check_invariants()


def test_state_rows_are_zero_when_a_slot_starts():
    cache = make({0: KV, 1: STATE}, max_slots=4)
    state = [g for g in cache.groups if g.need.kind == "state"][0].state
    assert state.shape == (1, 4, 3, 5)
    slot = cache.alloc_slot()
    state[0, slot] = 7.0
    cache.free_slot(slot)
    assert cache.alloc_slot() == slot and float(state[0, slot].abs().sum()) == 0.0
    view = cache.layer_cache(1, True, {})
    assert view.state.data_ptr() == state[0].data_ptr() and view.k_pages is None


def test_random_traffic_keeps_the_books_straight():
    rng = random.Random(7)
    cache = make({0: KV, 1: WINDOWED, 2: STATE}, max_tokens=64 * 40, max_slots=12)
    live = {}
    for _ in range(3000):
        action = rng.random()
        if action < 0.25 and len(live) < 12:
            live[cache.alloc_slot()] = 0
        elif action < 0.4 and live:
            slot = rng.choice(list(live))
            cache.free_slot(slot)
            del live[slot]
        elif live:
            chosen = rng.sample(list(live), rng.randint(1, len(live)))
            requests = [(slot, rng.choice([1, 1, 1, 5, 64, 130])) for slot in chosen]
            try:
                cache.reserve(requests)
            except CacheFull:
                for slot in chosen:
                    assert cache.length(slot) == live[slot]
            else:
                if rng.random() < 0.1:
                    cache.rollback(requests)
                else:
                    cache.commit(requests)
                    for slot, n in requests:
                        live[slot] += n
        cache.check_invariants()
        assert sorted(live) == cache.live_slots()
        for slot, length in live.items():
            assert cache.length(slot) == length
    for slot in list(live):
        cache.free_slot(slot)
    cache.check_invariants()
    assert cache.free_page_count() == 40 and cache.live_slots() == []
