"""The cache manager on the host: no page lost, held twice or freed twice, under random orders of
requests; windows give pages back; slots; all-or-nothing reservation."""
import random

import pytest

from pulse_infer_amd.cache import (CacheError, CacheManager, OutOfPages, PagedKVSpec, PageError, PagePool, StateSlots,
                                   StateSpec)


def test_pool_hands_out_each_page_once_and_reuses_the_last_freed_first():
    pool = PagePool(4)
    first = pool.allocate(3)
    assert len(set(first)) == 3 and pool.num_free == 1 and pool.num_held == 3
    with pytest.raises(OutOfPages):
        pool.allocate(2)
    assert pool.num_free == 1                      # all or nothing (reference: src/runtime/block_manager.cpp:44-46)
    pool.release([first[1]])
    assert pool.allocate(1) == [first[1]]          # last in, first out
    pool.check()
    with pytest.raises(PageError, match="twice"):
        pool.release([first[0], first[0]])
    assert pool.is_held(first[0])                  # a failed release changes nothing
    pool.release(first)
    with pytest.raises(PageError, match="twice"):
        pool.release([first[0]])
    with pytest.raises(PageError, match="not one of"):
        pool.release([99])
    assert pool.high_water == 3
    pool.check()


def test_slots():
    slots = StateSlots(2)
    a, b = slots.take("a"), slots.take("b")
    assert {a, b} == {0, 1}
    with pytest.raises(CacheError):
        slots.take("c")
    slots.give_back(a)
    assert slots.take("c") == a
    with pytest.raises(CacheError):
        slots.give_back(5)


FULL = PagedKVSpec(2, 16)
WIN = PagedKVSpec(2, 16, window=10)


def test_groups_by_need():
    m = CacheManager([FULL, WIN, FULL, None, StateSpec((3,)), WIN], page_size=4, num_pages=8, max_requests=2)
    assert len(m.groups) == 2
    assert m.groups[0].runs == [0, 2] and m.groups[1].runs == [1, 5]
    assert m.run_group[2] == (0, 1) and m.run_group[5] == (1, 1)
    assert list(m.state_runs) == [4]
    with pytest.raises(TypeError):
        CacheManager(["what"], 4, 8, 2)


def test_reserve_is_all_or_nothing_across_groups():
    m = CacheManager([FULL, WIN], page_size=4, num_pages=4, max_requests=3, group_pages={WIN: 2})
    m.add_request("a")
    m.reserve("a", 8)                              # 2 pages in each group: the window group is now full
    m.add_request("b")
    assert m.pages_needed("b", 5) == [2, 2] and not m.can_reserve("b", 5)
    with pytest.raises(OutOfPages):
        m.reserve("b", 5)
    assert m.table(0, "b") == [] and m.free_pages() == [2, 0]   # nothing was taken in the group that had room
    m.check()
    with pytest.raises(CacheError, match="already live"):
        m.add_request("a")
    with pytest.raises(CacheError, match="not live"):
        m.reserve("zz", 1)
    with pytest.raises(CacheError, match="reserved"):
        m.advance("a", 9)
    m.advance("a", 8)
    with pytest.raises(CacheError, match="go back"):
        m.advance("a", 3)


def test_window_pages_are_given_back_as_the_window_passes():
    m = CacheManager([WIN], page_size=4, num_pages=6, max_requests=1)
    m.add_request("r")
    held_max = 0
    for length in range(1, 60):
        m.reserve("r", length)
        m.advance("r", length)
        table = m.table(0, "r")
        # the next token sits at position `length` and reads keys > length - 10
        first_needed = max(0, length - 10 + 1)
        for i, page in enumerate(table):
            whole_page_dead = (i + 1) * 4 <= first_needed
            assert (page == -1) == whole_page_dead, (length, table)
        held_max = max(held_max, m.groups[0].pool.num_held)
        m.check()
    assert held_max <= 4                           # ceil((10 - 1) / 4) + 1 pages, however long the request
    m.free_request("r")
    assert m.groups[0].pool.num_free == 6


def test_a_stamp_tells_when_a_requests_tables_have_changed():
    """Who keeps a copy of a request's block tables (a recorded step's buffer) compares stamps: the stamp moves with
    every page taken and every page given back below a window, stays while a reservation fits the pages that are
    there, and is never that of another request, not even of a later one with the same name."""
    m = CacheManager([FULL, WIN], page_size=4, num_pages=12, max_requests=2)
    m.add_request("a")
    m.add_request("b")
    seen = {m.tables_stamp("a"), m.tables_stamp("b")}
    assert len(seen) == 2
    m.reserve("a", 3)
    first = m.tables_stamp("a")
    assert first not in seen and m.table(0, "a") != []
    seen.add(first)
    free = m.free_pages()
    for length in (4, 2, 4):                      # inside the page it has: nothing is taken, nothing changes
        assert m.can_reserve("a", length)
        m.reserve("a", length)
        assert m.tables_stamp("a") == first and m.free_pages() == free
    assert m.reserved("a") == 4
    m.reserve("a", 5)                             # a second page in both groups
    second = m.tables_stamp("a")
    assert second not in seen and m.free_pages() == [f - 1 for f in free]
    seen.add(second)
    m.reserve("a", 16)
    seen.add(m.tables_stamp("a"))
    m.advance("a", 8)                             # the window (10 keys) still reaches the first page
    before = m.tables_stamp("a")
    m.advance("a", 14)                            # now it does not: the window group's first page goes back
    assert m.table(1, "a")[0] == -1 and m.tables_stamp("a") != before and m.tables_stamp("a") not in seen
    seen.add(m.tables_stamp("a"))
    assert m.tables_stamp("b") in seen            # b was never touched
    m.free_request("a")
    m.add_request("a")
    assert m.tables_stamp("a") not in seen and not m.can_reserve("a", 4 * 12 + 1) and m.can_reserve("a", 4)
    m.check()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_every_page_accounted_for(seed):
    rng = random.Random(seed)
    m = CacheManager([FULL, WIN, FULL], page_size=4, num_pages=24, max_requests=5)
    live = {}
    next_id = 0
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and len(live) < 5:
            m.add_request(next_id)
            live[next_id] = 0
            next_id += 1
        elif action < 0.8 and live:
            rid = rng.choice(list(live))
            grow = rng.choice([1, 1, 1, 2, 5, 13])
            if m.can_reserve(rid, live[rid] + grow):
                before = m.free_pages()
                m.reserve(rid, live[rid] + grow)
                live[rid] += grow
                m.advance(rid, live[rid])
                assert all(a <= b for a, b in zip(m.free_pages(), [x + 4 for x in before]))
            else:
                with pytest.raises(OutOfPages):
                    m.reserve(rid, live[rid] + grow)
        elif live:
            rid = rng.choice(list(live))
            m.free_request(rid)
            del live[rid]
            with pytest.raises(CacheError):
                m.free_request(rid)                # freed twice
        m.check()
        for rid, length in live.items():
            assert m.computed(rid) == length
            assert len(m.table(0, rid)) == (length + 3) // 4
    for rid in list(live):
        m.free_request(rid)
    assert m.free_pages() == [24, 24] and m.slots.num_free == 5
    m.check()


def test_pages_are_used_again():
    m = CacheManager([FULL], page_size=4, num_pages=3, max_requests=2)
    m.add_request("a")
    m.reserve("a", 12)
    pages = list(m.table(0, "a"))
    m.free_request("a")
    m.add_request("b")
    m.reserve("b", 4)
    assert m.table(0, "b")[0] == pages[-1]         # the page freed last is handed out first
    m.reset()
    assert m.free_pages() == [3] and not m.requests
