"""Cache manager: pages, per-group block tables, windows, state slots."""

import random

import pytest

from tokensprint_amd.cache import (CacheManager, GroupLayout, OutOfPages, OutOfSlots, PagePool,
                                   StateSlots, group_runs, page_bytes)
from tokensprint_amd.parts.base import PagedKVNeed, SlotStateNeed

import torch


def manager(num_pages=8, page=4, windows=(None,), slots=4):
    groups = [GroupLayout(2, 16, w, (i,)) for i, w in enumerate(windows)]
    return CacheManager(groups, page, num_pages, slots)


def test_pool_fifo_and_double_free():
    pool = PagePool(3)
    a, b = pool.take("x"), pool.take("x")
    assert (a, b) == (0, 1)                       # taken from the left
    pool.give_back(a, "x")
    assert list(pool.free) == [2, 0]              # given back on the right
    with pytest.raises(RuntimeError, match="freed twice"):
        pool.give_back(a, "x")
    with pytest.raises(RuntimeError, match="owned by"):
        pool.give_back(b, "y")
    pool.check()


def test_slots():
    s = StateSlots(2)
    assert s.take("a") == 0 and s.take("b") == 1
    with pytest.raises(OutOfSlots):
        s.take("c")
    s.give_back(0, "a")
    assert s.take("c") == 0
    with pytest.raises(RuntimeError, match="owned by"):
        s.give_back(1, "c")


def test_growth_uses_the_tail_of_the_last_page():
    # the reference's can_append arithmetic (block_manager.py:290-322) at page size 4
    m = manager(num_pages=3)
    rc = m.admit("a")
    m.extend(rc, 8)
    assert rc.tables[0] == [0, 1] and m.pools[0].num_free == 1
    assert m.pages_needed(rc, 11) == [1]          # 8 % 4 == 0: no tail, one page for 3 tokens
    m.extend(rc, 11)
    assert m.pages_needed(rc, 12) == [0]          # tail of one fits the next token
    m.extend(rc, 12)
    assert m.pages_needed(rc, 13) == [1] and not m.can_extend(rc, 13)
    with pytest.raises(OutOfPages):
        m.extend(rc, 13)
    assert rc.num_tokens == 12 and len(rc.tables[0]) == 3     # nothing half done
    m.free(rc)
    assert m.pools[0].num_free == 3 and not m.live
    m.check()


def test_finish_gives_everything_back_and_pages_are_used_again():
    m = manager(num_pages=4)
    a = m.admit("a"); m.extend(a, 16)
    assert m.pools[0].num_free == 0
    b = m.admit("b")
    assert not m.can_extend(b, 1)
    m.free(a)
    m.extend(b, 9)
    assert sorted(b.tables[0]) == sorted(b.tables[0]) and len(b.tables[0]) == 3
    assert set(b.tables[0]) <= {0, 1, 2, 3}
    m.check()
    with pytest.raises(RuntimeError, match="not live"):
        m.free(a)


def test_window_group_gives_pages_back_as_the_window_passes():
    m = manager(num_pages=16, page=4, windows=(None, 6))
    rc = m.admit("a")
    m.extend(rc, 20)                 # one portion of 20: both groups hold 5 pages
    assert len(rc.tables[0]) == 5 and [p >= 0 for p in rc.tables[1]] == [True] * 5
    m.extend(rc, 21)                 # next query at 20 sees keys 15..20: pages 0..2 go back
    assert [p >= 0 for p in rc.tables[1]] == [False, False, False, True, True, True]
    assert all(p >= 0 for p in rc.tables[0])
    assert m.pools[1].num_used == 3 and m.pools[0].num_used == 6
    for n in range(22, 60):
        m.extend(rc, n)
        held = sum(p >= 0 for p in rc.tables[1])
        assert held <= 3             # ceil((6 + 4 - 1) / 4) + 1 at most
        first_visible = max(0, (n - 1) - 6 + 1)
        assert all(rc.tables[1][i] >= 0 for i in range(first_visible // 4, -(-n // 4)))
        m.check()
    m.free(rc)
    assert m.pools[0].num_used == 0 and m.pools[1].num_used == 0


def test_window_release_counts_toward_what_a_step_needs():
    m = manager(num_pages=3, page=4, windows=(5,))
    rc = m.admit("a")
    m.extend(rc, 12)
    assert m.pools[0].num_free == 0
    # the query at 12 sees keys 8..12: pages 0 and 1 go back before one is taken
    assert m.pages_needed(rc, 16) == [-1] and m.can_extend(rc, 16)
    m.extend(rc, 16)
    assert [p >= 0 for p in rc.tables[0]] == [False, False, True, True]
    m.check()


def test_groups_are_keyed_by_shape_and_window():
    needs = [PagedKVNeed(2, 16), PagedKVNeed(2, 16, 8), None, PagedKVNeed(2, 16),
             SlotStateNeed((4,)), PagedKVNeed(4, 16)]
    groups, group_of = group_runs(needs)
    assert [g.runs for g in groups] == [(0, 3), (1,), (5,)]
    assert group_of == {0: 0, 3: 0, 1: 1, 5: 2}
    assert page_bytes(groups, 4, torch.bfloat16) == (2 + 1) * 2 * 2 * 4 * 16 * 2 + 2 * 4 * 4 * 16 * 2


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_lose_nothing(seed):
    rnd = random.Random(seed)
    windows = (None, rnd.choice([3, 9, 17]))
    m = manager(num_pages=rnd.choice([6, 10, 24]), page=rnd.choice([1, 4, 16]),
                windows=windows, slots=3)
    live = {}
    for step in range(400):
        action = rnd.random()
        if action < 0.25 and len(live) < 3:
            rid = f"r{step}"
            live[rid] = m.admit(rid)
        elif action < 0.85 and live:
            rc = live[rnd.choice(sorted(live))]
            n = rc.num_tokens + rnd.choice([1, 1, 1, 2, 7, 30])
            if m.can_extend(rc, n):
                m.extend(rc, n)
            else:
                with pytest.raises(OutOfPages):
                    m.extend(rc, n)
        elif live:
            rid = rnd.choice(sorted(live))
            m.free(live.pop(rid))
        m.check()
        for pool in m.pools:
            assert pool.num_free + pool.num_used == pool.num_pages
    for rc in live.values():
        m.free(rc)
    m.check()
    assert all(p.num_used == 0 for p in m.pools) and m.slots.num_free == 3
    with pytest.raises(OutOfSlots):
        for i in range(4):
            m.admit(f"x{i}")
