"""Cache manager: the reference's block-manager behaviours
(tests/unit/test_block_manager.py:6-87), groups with windows, state slots, and
random request orders that must never lose, double-hold or double-free a page."""

import random

import pytest

from tokamak_amd.cache import (
    RELEASED, CacheGroupSpec, CacheManager, OutOfPagesError, OutOfSlotsError, PagePool, StateSlots,
)


def manager(num_pages=8, page_size=4, slots=8, groups=None):
    groups = groups or [CacheGroupSpec("full", (0, 1))]
    return CacheManager(groups, num_pages, page_size, slots)


def test_pages_needed_rounds_up():
    m = manager()
    assert [m.pages_needed(n) for n in (0, 1, 4, 5)] == [0, 1, 1, 2]


def test_invalid_construction():
    with pytest.raises(ValueError):
        manager(num_pages=0)
    with pytest.raises(ValueError):
        manager(page_size=0)
    with pytest.raises(ValueError):
        StateSlots(0)
    with pytest.raises(ValueError, match="two groups"):
        CacheManager([CacheGroupSpec("a", (0,)), CacheGroupSpec("b", (0,))], 4, 4, 2)


def test_growth_on_demand_idempotent_and_append_only():
    m = manager()
    m.ensure_capacity("a", 5)
    assert len(m.block_table("a")) == 2 and m.num_free_pages() == 6 and m.reserved_tokens("a") == 8
    before = list(m.block_table("a"))
    m.ensure_capacity("a", 5)
    assert m.block_table("a") == before
    m.ensure_capacity("a", 12)
    assert m.block_table("a")[:2] == before and len(m.block_table("a")) == 3


def test_lifo_lowest_first_and_reuse_order():
    m = manager(num_pages=4)
    m.ensure_capacity("a", 8)
    assert m.block_table("a") == [0, 1]       # lowest ids first
    m.free("a")
    m.ensure_capacity("b", 4)
    assert m.block_table("b") == [1]          # the page freed last is used again first


def test_requests_get_disjoint_pages():
    m = manager()
    m.ensure_capacity("a", 8)
    m.ensure_capacity("b", 8)
    assert not set(m.block_table("a")) & set(m.block_table("b"))


def test_exhaustion_raises_and_leaves_state_intact():
    m = manager(num_pages=4)
    m.ensure_capacity("a", 12)
    with pytest.raises(OutOfPagesError, match="1 of 4 are free"):
        m.ensure_capacity("b", 8)
    assert m.num_free_pages() == 1 and m.block_table("b") == []
    assert not m.can_hold("b", 8) and m.can_hold("b", 4)


def test_free_is_idempotent_and_pages_are_reusable():
    m = manager(num_pages=4)
    m.ensure_capacity("a", 16)
    assert m.num_free_pages() == 0
    m.free("a")
    m.free("a")
    m.free("never seen")
    assert m.num_free_pages() == 4 and m.block_table("a") == []
    m.ensure_capacity("b", 16)
    m.check()


def test_slack_is_less_than_one_page():
    m = manager(num_pages=64, page_size=16)
    for i, n in enumerate([1, 15, 16, 17, 100, 255]):
        m.ensure_capacity(i, n)
        assert 0 <= m.reserved_tokens(i) - n < 16


def test_pool_refuses_double_free_and_double_take():
    pool = PagePool(2)
    pages = pool.take(2)
    pool.give_back(pages)
    with pytest.raises(AssertionError, match="freed twice"):
        pool.give_back(pages[:1])


def test_groups_have_pools_and_tables_of_their_own():
    groups = [CacheGroupSpec("full", (0, 2)), CacheGroupSpec("window8", (1,), window=8)]
    m = CacheManager(groups, [8, 3], 4, 4)
    m.ensure_capacity("a", 10)
    assert len(m.block_table("a", 0)) == 3 and len(m.block_table("a", 1)) == 3
    assert m.num_free_pages(0) == 5 and m.num_free_pages(1) == 0
    assert m.group_of_slot == {0: 0, 2: 0, 1: 1}
    # all or nothing across groups: group 1 is exhausted, so group 0 must not grow either
    with pytest.raises(OutOfPagesError, match="window8"):
        m.ensure_capacity("a", 14)
    assert len(m.block_table("a", 0)) == 3
    m.check()


def test_window_group_gives_pages_back_while_running():
    groups = [CacheGroupSpec("full", (0,)), CacheGroupSpec("window8", (1,), window=8)]
    m = CacheManager(groups, [16, 4], 4, 4)
    m.ensure_capacity("a", 16)                      # 4 pages in both groups
    assert m.num_free_pages(1) == 0
    # next query sits at position 16 and sees 9..16: pages 0 and 1 (positions 0..7) are dead
    assert m.release_behind_window("a", 16) == 2
    assert m.block_table("a", 1)[:2] == [RELEASED, RELEASED]
    assert m.num_free_pages(1) == 2 and m.num_free_pages(0) == 12   # the full group keeps everything
    assert m.release_behind_window("a", 16) == 0    # idempotent
    assert m.release_behind_window("a", 12) == 0    # never moves backwards
    m.ensure_capacity("a", 20)                      # the window group reuses what it gave back
    assert m.reserved_tokens("a", 1) == 12
    m.ensure_capacity("b", 4)
    m.free("a")
    m.free("b")
    assert m.num_free_pages(0) == 16 and m.num_free_pages(1) == 4
    m.check()


def test_state_slots():
    s = StateSlots(2)
    assert s.acquire("a") == 0 and s.acquire("b") == 1 and s.acquire("a") == 0
    with pytest.raises(OutOfSlotsError):
        s.acquire("c")
    s.release("a")
    s.release("a")
    assert s.acquire("c") == 0 and s.slot_of("a") is None
    s.check()


@pytest.mark.parametrize("seed", range(5))
def test_random_orders_never_lose_or_share_a_page(seed):
    rng = random.Random(seed)
    groups = [CacheGroupSpec("full", (0,)), CacheGroupSpec("window12", (1,), window=12)]
    m = CacheManager(groups, [24, 10], 4, 5)
    lengths: dict[int, int] = {}
    next_id = 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.slots.num_free:
            m.admit(next_id)
            lengths[next_id] = 0
            next_id += 1
        elif op < 0.8 and lengths:
            r = rng.choice(list(lengths))
            grow = rng.choice([1, 1, 1, 2, 5, 9])
            m.release_behind_window(r, lengths[r])
            try:
                m.ensure_capacity(r, lengths[r] + grow)
                lengths[r] += grow
            except OutOfPagesError:
                victim = max(lengths)            # newest
                m.free(victim)
                del lengths[victim]
        elif lengths:
            r = rng.choice(list(lengths))
            m.free(r)
            del lengths[r]
        m.check()
        for r, n in lengths.items():
            assert len(m.block_table(r, 0)) == m.pages_needed(n)
            live = [p for p in m.block_table(r, 1) if p != RELEASED]
            assert len(live) <= m.pages_needed(12 + 9) + 1   # window plus the largest portion, plus an edge
    for r in list(lengths):
        m.free(r)
    m.check()
    assert m.num_free_pages(0) == 24 and m.num_free_pages(1) == 10 and m.slots.num_free == 5
