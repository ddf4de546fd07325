"""The cache manager: no page lost, held twice or freed twice, under random orders of
requests; windows give pages back; state slots."""
import numpy as np
import pytest
import torch
from hypothesis import given, settings, strategies as st

from wllm_amd.cache import CacheManager, CacheNeed, OutOfPages, OutOfSlots, PageAccountingError, PagePool


def manager(num_pages=8, page_size=4, window=None, max_requests=4, two_groups=False, **kw):
    needs = {0: CacheNeed(1, 8, window), 1: CacheNeed(1, 8, window)}
    if two_groups:
        needs[2] = CacheNeed(1, 8, None if window else 6)
    return CacheManager(needs, page_size, num_pages, max_requests, torch.float32, "cpu", **kw)


def test_pool_hands_out_the_page_freed_last():
    # the reference's allocator test (tests/test_kv_cache.py:12-23)
    pool = PagePool(4)
    a, b = pool.allocate("x"), pool.allocate("x")
    assert pool.num_free == 2
    pool.free(a, "x")
    assert pool.num_free == 3
    assert pool.allocate("y") == a
    assert a == 3 and b == 2     # the free list is handed out from its end


def test_pool_exhaustion_and_misuse_raise():
    pool = PagePool(1)
    p = pool.allocate("x")
    with pytest.raises(OutOfPages):
        pool.allocate("x")
    with pytest.raises(PageAccountingError):
        pool.free(p, "someone else")
    pool.free(p, "x")
    with pytest.raises(PageAccountingError):
        pool.free(p, "x")


def test_reserve_grows_the_table_at_page_boundaries():
    # tests/test_kv_cache.py:33-53
    m = manager()
    m.open(0)
    slots = m.reserve(0, 4)[0]
    table = m.block_table(0, 0)
    assert len(table) == 1 and slots.tolist() == [table[0] * 4 + i for i in range(4)]
    m.commit(0, 4)
    slots = m.reserve(0, 1)[0]
    assert len(m.block_table(0, 0)) == 2 and slots.tolist() == [m.block_table(0, 0)[1] * 4]
    assert m.reserve(0, 1)[0].tolist() == slots.tolist(), "reserve again before commit: the same answer"
    m.commit(0, 1)
    assert m.context_len(0) == 5
    m.check()


def test_close_gives_everything_back():
    m = manager(num_pages=2)
    m.open(0)
    m.reserve(0, 4)
    m.commit(0, 4)
    assert m.num_free_pages(0) == 1
    m.close(0)
    assert m.num_free_pages(0) == 2
    m.check()


def test_reserve_is_all_or_nothing():
    m = manager(num_pages=3)
    m.open("a")
    m.open("b")
    m.reserve("a", 8)
    m.commit("a", 8)
    with pytest.raises(OutOfPages):
        m.reserve("b", 8)
    assert m.num_free_pages(0) == 1 and m.block_table("b", 0) == []
    m.check()


def test_trim_gives_back_what_an_abandoned_step_took():
    m = manager(num_pages=4)
    m.open("a")
    m.reserve("a", 3)
    m.commit("a", 3)
    m.reserve("a", 9)
    assert m.num_free_pages(0) == 1
    m.trim("a")
    assert m.num_free_pages(0) == 3 and len(m.block_table("a", 0)) == 1
    m.check()


def test_groups_have_pools_of_their_own():
    m = manager(two_groups=True)
    assert len(m.groups) == 2 and m.groups[0].entries == [0, 1] and m.groups[1].entries == [2]
    assert m.entry_storage(0).shape == (8, 2, 1, 32)
    m.open("a")
    both = m.reserve("a", 6)
    assert len(both) == 2
    m.commit("a", 6)
    assert m.num_free_pages(0) == 6 and m.num_free_pages(1) == 6
    m.check()


def test_window_gives_pages_back_once_passed_and_they_are_used_again():
    m = manager(num_pages=4, page_size=4, window=6)
    m.open("a")
    for _ in range(40):
        m.reserve("a", 1)
        m.commit("a", 1)
        m.check()
        held = [p for p in m.block_table("a", 0) if p >= 0]
        # a query at position ctx reaches back to ctx - 5: at most 3 pages
        assert len(held) <= 3
    table = m.block_table("a", 0)
    assert table[:8] == [-1] * 8 and len(set(p for p in table if p >= 0)) == len([p for p in table if p >= 0])
    ctx = m.context_len("a")
    first_needed = (ctx - 6 + 1) // 4
    assert all(p >= 0 for p in table[first_needed:])
    m.close("a")
    assert m.num_free_pages(0) == 4


def test_pages_for_bounds_a_window():
    m = manager(num_pages=64, page_size=4, window=6)
    assert m.pages_for(0, 100, 1) == 3 and m.pages_for(0, 5, 1) == 2
    full = manager(num_pages=64, page_size=4)
    assert full.pages_for(0, 100, 1) == 25 and full.pages_for(0, 4, 1) == 1


def test_state_slots_are_zeroed_unique_and_bounded():
    m = CacheManager({0: CacheNeed(1, 8)}, 4, 4, 2, torch.float32, "cpu", state_shapes={0: (3,)})
    a = m.open("a")
    m.state[0][a] = 5.0
    b = m.open("b")
    assert a != b
    with pytest.raises(OutOfSlots):
        m.open("c")
    m.close("a")
    assert m.open("c") == a and m.state[0][a].abs().sum() == 0, "a slot handed out again is zeroed"
    with pytest.raises(KeyError):
        m.open("c")
    m.check()


def test_poisoned_pages_show_stale_reads():
    m = manager(num_pages=2, poison_freed_pages=True)
    m.open("a")
    m.reserve("a", 4)
    page = m.block_table("a", 0)[0]
    m.close("a")
    assert torch.isnan(m.entry_storage(0)[page]).all() and torch.isnan(m.entry_storage(1)[page]).all()


@settings(max_examples=60, deadline=None)
@given(st.lists(st.tuples(st.integers(0, 5), st.integers(0, 3), st.integers(1, 9)), min_size=1, max_size=80),
       st.sampled_from([None, 5, 11]), st.integers(3, 12))
def test_no_page_is_lost_or_held_twice_under_random_orders(ops_list, window, num_pages):
    """Random opens, reserves, commits, abandoned reserves and closes of up to six requests."""
    m = manager(num_pages=num_pages, page_size=4, window=window, max_requests=6, two_groups=True)
    for rid, action, n in ops_list:
        if not m.is_open(rid):
            m.open(rid)
            continue
        if action == 3:
            m.close(rid)
        else:
            free_before = [m.num_free_pages(g) for g in range(2)]
            try:
                slots = m.reserve(rid, n)
            except OutOfPages:
                assert [m.num_free_pages(g) for g in range(2)] == free_before, "a refused reserve takes nothing"
            else:
                ctx = m.context_len(rid)
                for g in range(2):
                    table = m.block_table(rid, g)
                    want = [table[(ctx + i) // 4] * 4 + (ctx + i) % 4 for i in range(n)]
                    assert slots[g].tolist() == want
                if action == 2:
                    m.trim(rid)
                else:
                    m.commit(rid, n)
        m.check()
        for g, grp in enumerate(m.groups):
            held = sum(1 for rc in m.requests.values() for p in rc.tables[g] if p >= 0)
            assert held + grp.pool.num_free == grp.pool.num_pages
            if grp.need.window is None:
                for rid2, rc in m.requests.items():
                    assert len(rc.tables[g]) >= -(-rc.context_len // 4)
    for rid in list(m.requests):
        m.close(rid)
    assert all(g.pool.num_free == g.pool.num_pages for g in m.groups)
