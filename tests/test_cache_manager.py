"""The cache manager's page accounting: no page lost, held twice or freed twice,
under random orders of requests; window groups give pages back and never hold more
than the window needs; reservation is all-or-nothing."""

import random

import pytest
import torch

from cwm_amd.cache import CacheManager, OutOfPages, PageAccountingError, PagePool, first_page_needed
from cwm_amd.parts import PagedKVSpec, StateSpec


def specs(window=8):
    return [PagedKVSpec(1, 32, window), PagedKVSpec(1, 32, window), PagedKVSpec(1, 32, None), StateSpec((4,)), None]


def test_pool_hands_out_lowest_first_and_catches_double_free():
    pool = PagePool(4)
    assert [pool.take() for _ in range(4)] == [0, 1, 2, 3]
    with pytest.raises(OutOfPages):
        pool.take()
    pool.give(2)
    pool.give(0)
    assert pool.take() == 0 and pool.take() == 2
    pool.give(1)
    with pytest.raises(PageAccountingError):
        pool.give(1)
    with pytest.raises(PageAccountingError):
        pool.give(9)


def test_groups_by_retention_need():
    m = CacheManager(specs(), page_size=4, num_pages=10, max_requests=3)
    assert [g.window for g in m.groups] == [8, None]
    assert m.groups[0].cache_ids == [0, 1] and m.groups[1].cache_ids == [2]
    assert m.state_caches == [3]
    m2 = CacheManager(specs(), page_size=4, num_pages={8: 5, None: 20}, max_requests=3)
    assert [g.pool.num_pages for g in m2.groups] == [5, 20]


def test_first_page_needed():
    assert first_page_needed(100, None, 4) == 0
    assert first_page_needed(7, 8, 4) == 0  # a query at position 7 reads keys 0..7
    assert first_page_needed(11, 8, 4) == 1  # position 11 reads 4..11
    assert first_page_needed(12, 8, 4) == 1  # position 12 reads 5..12
    assert first_page_needed(15, 8, 4) == 2  # position 15 reads 8..15


def test_window_group_gives_pages_back_and_global_keeps_them():
    m = CacheManager(specs(window=8), page_size=4, num_pages=64, max_requests=2)
    m.admit("a")
    n = 0
    for step in (5, 3, 1, 1, 9, 2, 16, 1, 1, 1):
        assert m.extend("a", step)
        during = m.pages_held("a")
        # while the step runs, pages from the first needed one of the old length to the new end are held
        lo = first_page_needed(n, 8, 4)
        hi = (n + step - 1) // 4
        assert during[0] == hi - lo + 1
        m.advance("a", step)
        n += step
        held = m.pages_held("a")
        assert held[1] == (n + 3) // 4
        assert held[0] == (n + 3) // 4 - first_page_needed(n, 8, 4)
        assert held[0] <= (8 - 1 + 3) // 4 + 1
        m.check()
    table = m.table(0, "a")
    assert all(p == -1 for p in table[: first_page_needed(n, 8, 4)])
    m.release("a")
    m.check()
    assert m.free_pages() == [64, 64]


def test_extend_is_all_or_nothing():
    m = CacheManager(specs(), page_size=4, num_pages={8: 2, None: 10}, max_requests=2)
    m.admit("a")
    before = m.free_pages()
    assert not m.extend("a", 12)  # the window group has 2 pages, 3 are needed at once
    assert m.free_pages() == before and m.pages_held("a") == [0, 0]
    assert m.extend("a", 8)
    m.advance("a", 8)
    # a query at position 8 still reads key 1, so page 0 stays and no third page exists
    assert not m.extend("a", 4)
    assert m.pages_held("a") == [2, 2]
    m.check()


def test_advance_without_pages_is_an_error():
    m = CacheManager(specs(), page_size=4, num_pages=8, max_requests=1)
    m.admit("a")
    with pytest.raises(PageAccountingError):
        m.advance("a", 3)
    with pytest.raises(OutOfPages):
        m.admit("b")
    with pytest.raises(KeyError):
        m.admit("a")


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_keep_the_accounts(seed):
    rng = random.Random(seed)
    page_size = rng.choice([1, 4, 16])
    m = CacheManager(specs(window=rng.choice([3, 8, 40])), page_size=page_size, num_pages=rng.randrange(6, 40), max_requests=4)
    live = {}
    handed = {g.index: {} for g in m.groups}
    next_id = 0
    for _ in range(600):
        roll = rng.random()
        if roll < 0.25 and len(live) < 4:
            rid = f"r{next_id}"
            next_id += 1
            m.admit(rid)
            live[rid] = 0
        elif roll < 0.85 and live:
            rid = rng.choice(sorted(live))
            n = rng.choice([1, 1, 1, 2, 5, 17])
            free_before = m.free_pages()
            if m.extend(rid, n):
                for g in m.groups:
                    for lp, page in enumerate(m.table(g.index, rid)):
                        if page >= 0:
                            handed[g.index][page] = handed[g.index].get(page, set()) | {(rid, lp)}
                m.advance(rid, n)
                live[rid] += n
                assert m.length(rid) == live[rid]
            else:
                assert m.free_pages() == free_before
        elif live:
            rid = rng.choice(sorted(live))
            m.release(rid)
            del live[rid]
        m.check()
    for rid in list(live):
        m.release(rid)
    m.check()
    assert m.free_pages() == [g.pool.num_pages for g in m.groups]
    # pages were used again by other owners
    assert any(len(owners) > 1 for pages in handed.values() for owners in pages.values())


def test_another_retention_rule_needs_no_change_to_the_manager():
    """A cache need defined here, outside the framework: the first `sinks` keys are read by
    every query, beside a window.  The manager keeps their pages, gives back what lies
    between them and the window, groups the slot apart from a plain window of the same
    length, and the scheduler's and the step's questions are answered by the same methods."""
    from dataclasses import dataclass

    from cwm_amd.engine.batch import BatchError, Portion, build_batch

    @dataclass(frozen=True)
    class PinnedStartSpec(PagedKVSpec):
        sinks: int = 0

        def retention(self):
            return ("pinned start", self.sinks, self.window)

        def pinned_keys(self):
            return self.sinks

    page = 4
    specs_ = [
        PinnedStartSpec(n_kv_heads=1, head_dim=16, window=8, sinks=5),
        PagedKVSpec(n_kv_heads=1, head_dim=16, window=8),
        PinnedStartSpec(n_kv_heads=1, head_dim=16, window=8, sinks=5),
    ]
    m = CacheManager(specs_, page_size=page, num_pages={("pinned start", 5, 8): 12, 8: 12}, max_requests=2)
    assert [g.cache_ids for g in m.groups] == [[0, 2], [1]]
    pinned, plain = m.groups
    assert pinned.pinned_pages(page) == 2 and plain.pinned_pages(page) == 0
    # a request of 1,000 tokens with steps of 6: 2 pinned pages + ceil((7 + 6) / 4) + 1 of slack
    assert pinned.most_pages(1000, 6, page) == 2 + 4 + 1
    assert plain.most_pages(1000, 6, page) == 4 + 1
    assert pinned.most_pages(9, 6, page) == 3

    m.admit("a")
    for _ in range(10):
        assert m.extend("a", 3)
        m.advance("a", 3)
        m.check()
    # 30 tokens: the window's first key is 23, in page 5; pages 0 and 1 hold the pinned keys
    assert [p >= 0 for p in m.table(pinned.index, "a")] == [True, True, False, False, False, True, True, True]
    assert [p >= 0 for p in m.table(plain.index, "a")] == [False, False, False, False, False, True, True, True]
    assert m.free_pages() == [12 - 5, 12 - 3]

    # the step's check of the tables asks for the pinned pages too
    assert m.extend("a", 1)
    build_batch([Portion("a", [1], [0])], m, torch.device("cpu"), vocab_size=10)
    m.table(pinned.index, "a")[1] = -1
    with pytest.raises(BatchError, match="holds no page"):
        build_batch([Portion("a", [1], [0])], m, torch.device("cpu"), vocab_size=10)
    m.table(pinned.index, "a")[1] = 1
    m.release("a")
    m.check()
    assert m.free_pages() == [12, 12]
