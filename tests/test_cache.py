"""The cache manager on the CPU: no page lost, held twice or freed twice, under
random orders of requests; windows give pages back; reservations are all or
nothing."""
import random

import numpy as np
import pytest

from ninfer_amd.cache import CacheManager, OutOfPages, PageAllocator
from ninfer_amd.parts import CacheNeed


def test_allocator_is_lifo_and_counts_reuse():
    a = PageAllocator(4)
    p = a.alloc(3)
    assert p == [0, 1, 2] and a.free_pages == 1
    a.free([1])
    assert a.alloc(1) == [1] and a.reused == 1        # the page just given back comes first
    with pytest.raises(OutOfPages):
        a.alloc(2)
    assert a.free_pages == 1, "a failed allocation takes nothing"
    with pytest.raises(RuntimeError, match="not held"):
        a.free([3])
    a.free([0])
    with pytest.raises(RuntimeError, match="not held"):
        a.free([0])
    a.check()


def manager(num_pages=16, window=None, page_size=4, seqs=4, max_context=64):
    needs = [CacheNeed.keys_values(2, 8, None), CacheNeed.keys_values(2, 8, window)]
    return CacheManager(needs, page_size, num_pages, seqs, max_context, state_floats=0)


def test_groups_by_window():
    m = manager(window=8)
    assert [g.window for g in m.groups] == [None, 8]
    assert m.group_of_instance == {0: 0, 1: 1}
    same = CacheManager([CacheNeed.keys_values(2, 8), CacheNeed.keys_values(4, 16), None], 4, 8, 2, 32)
    assert len(same.groups) == 1 and same.groups[0].instances == [0, 1]
    assert same.kv_bytes_per_token(2) == 2 * (2 * 8 + 4 * 16) * 2


def test_groups_by_page_size():
    """Mixers that ask for pages of another size form groups of their own, with as many pages
    as hold the same number of tokens and tables as wide as the longest request needs."""
    needs = [CacheNeed.keys_values(2, 8), CacheNeed.keys_values(2, 8, None, page_size=8),
             CacheNeed.keys_values(2, 8, 6, page_size=8), CacheNeed.keys_values(1, 4, None, page_size=4)]
    m = CacheManager(needs, 4, 10, 3, 30)
    assert [(g.window, g.page_size, g.allocator.num_pages, g.max_pages) for g in m.groups] == \
        [(None, 4, 10, 8), (None, 8, 5, 4), (6, 8, 5, 4)]
    assert m.group_of_instance == {0: 0, 1: 1, 2: 2, 3: 0}
    s = m.acquire()
    assert m.pages_needed(s, 9) == [3, 2, 2]
    m.reserve(s, 9)
    m.commit(s, 9)
    assert m.block_table(0, [s]).tolist() == [[0, 1, 2]] and m.block_table(1, [s]).tolist() == [[0, 1]]
    m.reserve(s, 17)
    m.commit(s, 17)                       # the window of 6 has passed positions 0..7: one page of 8
    assert m.block_table(2, [s]).tolist() == [[-1, 1, 2]] and m.groups[2].window_freed == 1
    t = m.acquire()
    with pytest.raises(OutOfPages):
        m.reserve(t, 24)                  # 6 pages of 4 are wanted, 5 are free
    assert m.pages_free(1) == 2 and m.block_table(1, [t]).tolist() == [[-1]]
    m.check()
    with pytest.raises(ValueError, match="pages of 0"):
        CacheManager([CacheNeed.keys_values(2, 8, None, page_size=0)], 4, 10, 3, 30)


def test_reserve_commit_release_and_block_table():
    m = manager()
    s = m.acquire()
    m.reserve(s, 9)                                   # 3 pages of 4
    assert m.block_table(0, [s]).tolist() == [[0, 1, 2]]
    m.commit(s, 9)
    m.reserve(s, 10)                                  # still page 2
    assert m.pages_free(0) == 13
    t = m.acquire()
    m.reserve(t, 4)
    bt = m.block_table(0, [t, s], width=5)
    assert bt.dtype == np.int32 and bt.tolist() == [[3, -1, -1, -1, -1], [0, 1, 2, -1, -1]]
    m.release(s)
    assert m.pages_free(0) == 15
    u = m.acquire()
    m.reserve(u, 8)
    assert m.block_table(0, [u]).tolist() == [[2, 1]], "freed pages are used again first"
    assert m.pages_reused() == 2
    m.check()
    m.release(u)
    with pytest.raises(RuntimeError, match="not held"):
        m.release(u)


def test_reservation_is_all_or_nothing():
    m = manager(num_pages=4)
    a, b = m.acquire(), m.acquire()
    m.reserve(a, 8)
    with pytest.raises(OutOfPages):
        m.reserve_all([(a, 12), (b, 12)])             # needs 1 + 3 pages, 2 are free
    assert m.pages_free(0) == 2 and m.block_table(0, [b]).tolist() == [[-1]]
    with pytest.raises(OutOfPages, match="max_context"):
        m.reserve(a, 65)
    m.check()


def test_window_gives_pages_back_as_it_passes():
    m = manager(window=6, page_size=4, num_pages=8)
    s = m.acquire()
    for n in range(1, 30):
        m.reserve(s, n)
        m.commit(s, n)
        table = m.groups[1].tables[s]
        lowest_needed = max(0, n - 6 + 1)             # the next query is at position n
        for p, page in enumerate(table):
            last = (p + 1) * 4 - 1
            if last < lowest_needed:
                assert page == -1, f"page {p} should be back at length {n}"
            else:
                assert page >= 0
        assert all(p >= 0 for p in m.groups[0].tables[s]), "the full group keeps everything"
        m.check()
    assert m.groups[1].window_freed > 0
    assert m.groups[1].allocator.in_use <= 3          # ceil(6 / 4) + 1 pages at most
    m.release(s)
    assert m.pages_free(0) == 8 and m.pages_free(1) == 8


def test_state_bytes_are_reported_apart_from_the_pages():
    m = CacheManager([CacheNeed.keys_values(2, 8), None], 4, 8, 3, 32, state_floats=10)
    assert m.state_bytes_per_request() == 40 and m.kv_bytes_per_token(2) == 2 * 2 * 8 * 2
    assert manager().state_bytes_per_request() == 0


def test_slots_run_out_and_come_back():
    m = manager(seqs=2)
    a, b = m.acquire(), m.acquire()
    with pytest.raises(RuntimeError, match="slots"):
        m.acquire()
    m.release(a)
    assert m.acquire() == a and m.length(a) == 0


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_of_requests(seed):
    rng = random.Random(seed)
    if seed < 6:
        m = manager(num_pages=24, window=10, page_size=4, seqs=5, max_context=80)
    else:                                 # groups with pages of 4, 8 and 2 tokens
        needs = [CacheNeed.keys_values(2, 8), CacheNeed.keys_values(2, 8, 10, page_size=8),
                 CacheNeed.keys_values(2, 8, None, page_size=2)]
        m = CacheManager(needs, 4, 24, 5, 80)
    live = {}
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and m.free_slots:
            live[m.acquire()] = 0
        elif action < 0.85 and live:
            s = rng.choice(list(live))
            n = live[s] + rng.choice([1, 1, 1, 2, 5, 13])
            try:
                m.reserve(s, n)
            except OutOfPages:
                m.check()
                continue
            m.commit(s, n)
            live[s] = n
        elif live:
            s = rng.choice(list(live))
            m.release(s)
            del live[s]
        m.check()
        for s, n in live.items():
            assert m.length(s) == n
            full = m.groups[0].tables[s]
            assert len(full) >= -(-n // 4) and all(p >= 0 for p in full)
    for s in list(live):
        m.release(s)
    m.check()
    for g in m.groups:
        assert g.allocator.in_use == 0 and g.allocator.allocated == g.allocator.freed
