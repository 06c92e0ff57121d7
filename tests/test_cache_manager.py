"""The cache manager on the CPU: no page lost, held twice or freed twice, under random orders."""
import random

import numpy as np
import pytest

from kv_cache_optimization_for_llm_amd.cache.allocators import (BuddyAllocator, CacheAccountingError,
                                                                PagePool)
from kv_cache_optimization_for_llm_amd.cache.manager import CacheManager
from kv_cache_optimization_for_llm_amd.parts.base import StateSpec, attention_cache_spec

FULL = attention_cache_spec(2, 16)
WIN = attention_cache_spec(1, 32, kind="window", window=40)


def test_pool_is_lifo_and_counts_references():
    p = PagePool(6)
    a = p.take(3)
    assert a == [0, 1, 2] and p.free_count == 3 and p.accounting_holds()
    assert p.take(4) is None and p.free_count == 3        # all or nothing
    p.drop([1])
    assert p.take(1) == [1] and p.reuses == 1             # the page just freed goes out first
    p.share(2)
    assert p.drop([2]) == 0 and p.refcount(2) == 1        # still held by the other holder
    assert p.drop([2]) == 1 and p.refcount(2) == 0
    with pytest.raises(CacheAccountingError):
        p.drop([2])                                       # freed twice
    with pytest.raises(CacheAccountingError):
        p.share(5)                                        # never taken
    with pytest.raises(CacheAccountingError):
        p.drop([99])
    assert p.accounting_holds()


def test_buddy_rounds_splits_and_merges():
    b = BuddyAllocator(64)
    assert b.free_runs() == [(0, 64)]
    s1 = b.alloc(5)                   # rounds to 8
    assert s1 == 0 and b.round(5) == 8 and b.free_units == 56
    s2 = b.alloc(16)
    assert s2 % 16 == 0
    b.free(s1, 5)
    b.free(s2, 16)
    assert b.free_runs() == [(0, 64)] and b.free_units == 64 and b.reserved_units == 0
    with pytest.raises(CacheAccountingError):
        b.free(s1, 5)                 # freed twice


def test_buddy_pool_that_is_no_power_of_two_never_hands_out_the_end():
    b = BuddyAllocator(100)           # tree over 128; 100..127 are never free
    assert sum(n for _, n in b.free_runs()) == 100
    got = []
    while True:
        s = b.alloc(4)
        if s < 0:
            break
        assert 0 <= s and s + 4 <= 100
        got.append(s)
    assert len(got) == 25 and len(set(got)) == 25
    for s in got:
        b.free(s, 4)
    assert sum(n for _, n in b.free_runs()) == 100 and b.free_runs()[0] == (0, 64)


def test_buddy_counts_fragmentation_only_when_enough_is_free():
    b = BuddyAllocator(16)
    runs = [b.alloc(4) for _ in range(4)]
    assert b.alloc(4) == -1 and b.fragmentation_failures == 0     # simply full
    b.free(runs[0], 4)
    b.free(runs[2], 4)
    assert b.free_units == 8 and b.alloc(8) == -1 and b.fragmentation_failures == 1


def make(mode="paged", pages=32, seqs=4, specs=((FULL, [0, 1]),), states=None, page=16, max_len=256):
    return CacheManager(list(specs), states or {}, page_size=page, num_pages=pages, max_seqs=seqs,
                        max_seq_len=max_len, mode=mode)


def test_pages_follow_growth_and_return_at_the_end():
    m = make()
    s = m.admit("a")
    assert s == 0 and m.pages_needed(s, 1) == [1] and m.pages_needed(s, 16) == [1] and m.pages_needed(s, 17) == [2]
    assert m.grow(s, 33) and m.groups[0].free_pages() == 29
    assert m.pages_needed(s, 48) == [0] and m.pages_needed(s, 49) == [1]
    slots = m.slot_mapping(s, 14, 4, 0)
    row = m.groups[0].table_host[s]
    assert list(slots) == [row[0] * 16 + 14, row[0] * 16 + 15, row[1] * 16, row[1] * 16 + 1]
    m.commit(s, 33)
    m.check()
    m.free(s)
    assert m.groups[0].free_pages() == 32 and (m.groups[0].table_host == -1).all() and m.free_seats == 4
    m.check()


def test_growth_is_all_or_nothing_across_groups():
    m = make(pages=4, specs=((FULL, [0]), (WIN, [1])))
    a, b = m.admit("a"), m.admit("b")
    assert m.grow(a, 48)                                  # 3 pages in each group
    assert not m.can_grow(b, 32) and not m.grow(b, 32)    # 2 needed, 1 free
    assert [g.free_pages() for g in m.groups] == [1, 1]   # nothing taken by the failed growth
    assert m.grow(b, 16)
    m.check()


def test_window_group_gives_back_pages_the_window_has_passed():
    m = make(pages=8, specs=((FULL, [0]), (WIN, [1])))    # window 40, page 16
    s = m.admit("a")
    for n in range(1, 129):
        assert m.grow(s, n)
        m.commit(s, n)
        m.check()
        full, win = m.groups
        assert full.num_pages - full.free_pages() == (n + 15) // 16
        # next query at position n reads keys n-39..n: blocks below (n-39)//16 are gone
        keep_from = max(0, n - 39) // 16
        held = (n + 15) // 16 - keep_from
        assert win.num_pages - win.free_pages() == held and held <= 4
        assert (win.table_host[s, :keep_from] == -1).all()
    m.free(s)
    m.check()
    assert all(g.free_pages() == 8 for g in m.groups)
    assert m.groups[1].pool.reuses > 0                    # freed pages were used again


def test_no_seat_and_capacity_limits():
    m = make(seqs=2, max_len=40)
    a, b = m.admit("a"), m.admit("b")
    assert (a, b) == (0, 1) and m.admit("c") is None
    assert m.capacity_tokens(a) == 40 and not m.grow(a, 41) and m.grow(a, 40)
    m.free(a)
    assert m.admit("c") == 0                              # lowest free seat first


def test_contiguous_mode_reserves_runs_and_counts_fragmentation():
    m = make(mode="contiguous", pages=16, seqs=8)
    a = m.admit("a", reserve_tokens=40)                   # 3 pages -> run of 4
    assert m.capacity_tokens(a) == 64
    row = m.groups[0].table_host[a]
    assert list(row[:4]) == [row[0], row[0] + 1, row[0] + 2, row[0] + 3] and row[0] % 4 == 0
    assert m.grow(a, 64) and not m.grow(a, 65)
    b = m.admit("b", reserve_tokens=64)
    c = m.admit("c", reserve_tokens=64)
    d = m.admit("d", reserve_tokens=64)
    assert None not in (b, c, d) and m.admit("e", reserve_tokens=16) is None
    m.check()
    m.free(a)
    m.free(c)
    assert m.admit("f", reserve_tokens=128) is None       # 8 pages are free, but not in one run
    assert m.stats()["fragmentation_failures"] == 1
    st = m.stats()
    assert st["kv_tokens_reserved"] == 8 * 16 and st["kv_tokens_total"] == 16 * 16
    m.check()


def test_state_slots_are_part_of_the_books():
    m = make(states={0: StateSpec((4,))})
    assert m.state_specs[0].shape == (4,)


@pytest.mark.parametrize("mode", ["paged", "contiguous"])
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_orders_keep_the_books(mode, seed):
    rng = random.Random(seed)
    specs = ((FULL, [0, 1, 2]), (WIN, [3]))
    m = make(mode=mode, pages=24, seqs=5, specs=specs, max_len=200)
    live = {}
    admitted = refused = 0
    for it in range(600):
        op = rng.random()
        if op < 0.25 and len(live) < 5:
            rid = f"r{it}"
            seat = m.admit(rid, reserve_tokens=rng.choice([20, 50, 100, 200]))
            if seat is None:
                refused += 1
            else:
                assert seat not in live.values()
                live[rid] = seat
                admitted += 1
        elif op < 0.85 and live:
            rid = rng.choice(list(live))
            seat = live[rid]
            new_len = m.length(seat) + rng.choice([1, 1, 1, 2, 7, 16, 33])
            if m.can_grow(seat, new_len):
                assert m.grow(seat, new_len)
                for g in range(len(m.groups)):
                    slots = m.slot_mapping(seat, m.length(seat), new_len - m.length(seat), g)
                    assert (slots >= 0).all() and (slots < 24 * 16).all()
                m.commit(seat, new_len)
            else:
                before = [g.free_pages() for g in m.groups]
                assert not m.grow(seat, new_len)
                assert before == [g.free_pages() for g in m.groups]
        elif live:
            rid = rng.choice(list(live))
            m.free(live.pop(rid))
        m.check()
        # no page is held by two seats
        for g in m.groups:
            rows = g.table_host[g.table_host >= 0]
            assert len(rows) == len(set(rows.tolist()))
    for seat in live.values():
        m.free(seat)
    m.check()
    assert all(g.free_pages() == 24 for g in m.groups) and m.free_seats == 5
    assert admitted > 20


def test_a_sequence_cannot_grow_past_the_longest_length_inside_its_last_page():
    """The longest sequence need not be a multiple of the page size: the last page then has rows
    that must never be used, also on the quick path that skips the books when a page is there."""
    m = CacheManager([(attention_cache_spec(2, 16), [0])], {}, page_size=16, num_pages=8, max_seqs=2, max_seq_len=53)
    seat = m.admit("r")
    assert m.grow(seat, 50) and m.capacity_tokens(seat) == 53
    m.commit(seat, 50)
    assert m.pages_needed(seat, 53) == [0] and m.grow(seat, 53)
    assert not m.grow(seat, 54) and not m.can_grow(seat, 54)
    m.commit(seat, 53)
    assert not m.grow(seat, 54)
    m.check()
