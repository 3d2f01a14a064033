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
    a, b = pool.take(), pool.take()
    assert (a, b) == (0, 1)                       # taken from the left
    pool.give_back(a)
    assert list(pool.free) == [2, 0]              # given back on the right
    with pytest.raises(RuntimeError, match="freed twice"):
        pool.give_back(a)
    pool.take_tagged(b)                           # a second holder
    pool.give_back(b)
    assert pool.num_free == 2 and pool.refs[b] == 1
    pool.give_back(b)
    assert list(pool.free) == [2, 0, 1]
    pool.take_tagged(0)                           # a particular free page, out of order
    assert list(pool.free) == [2, 1] and pool.refs[0] == 1
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


def test_shrink_undoes_an_extend():
    from tokensprint_amd.parts.base import PagedKVNeed
    groups, _ = group_runs([PagedKVNeed(2, 16, None), PagedKVNeed(2, 16, 8)])
    m = CacheManager(groups, page_size=4, num_pages=12, num_slots=2)
    rc = m.admit("a")
    m.extend(rc, 9)
    held = [list(t) for t in rc.tables]
    free = [p.num_free for p in m.pools]
    m.extend(rc, 18)                      # takes pages in both groups, the window lets one go
    m.shrink(rc, 9)
    assert rc.num_tokens == 9 and [len(t) for t in rc.tables] == [3, 3]
    assert rc.tables[0] == held[0]
    assert m.pools[0].num_free == free[0] and m.pools[1].num_free >= free[1]
    m.check()
    m.extend(rc, 10)                      # and goes on as if nothing had happened
    m.check()
    with pytest.raises(ValueError, match="cannot shrink"):
        m.shrink(rc, 11)
    m.free(rc)
    assert all(p.num_used == 0 for p in m.pools)


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


# ------------------------------------------------------------------ prefix cache
def test_prefix_cache_reuses_full_pages_but_never_the_last():
    m = manager(num_pages=12, page=4)
    m.enable_prefix_cache()
    tokens = list(range(100, 118))                 # 18 tokens: pages 0..3 full, page 4 partial
    a = m.admit("a", tokens)
    assert a.num_tokens == 0                       # nothing cached yet
    m.extend(a, 18)
    m.register_full_pages(a, tokens, 18)
    assert len(a.hashes) == 4 and len(m.prefix_index) == 4
    # same prompt while "a" is live: its four full pages are shared
    b = m.admit("b", tokens)
    assert b.num_tokens == 16 and b.tables[0] == a.tables[0][:4]
    assert [m.pools[0].refs[p] for p in b.tables[0]] == [2, 2, 2, 2]
    m.extend(b, 18)
    assert b.tables[0][4] != a.tables[0][4]        # the partial page is its own
    m.check()
    # a prompt of exactly 16 tokens may take only three pages: its last token is computed
    c = m.admit("c", tokens[:16])
    assert c.num_tokens == 12
    m.free(c)
    # another continuation shares only the common full pages
    other = tokens[:8] + [7] * 10
    d = m.admit("d", other)
    assert d.num_tokens == 8 and d.tables[0] == a.tables[0][:2]
    m.free(d); m.free(b); m.free(a)
    assert m.pools[0].num_used == 0
    # freed pages keep their contents until they are handed out for something else
    e = m.admit("e", tokens)
    assert e.num_tokens == 16
    m.free(e)
    m.check()


def test_prefix_cache_forgets_evicted_pages_and_needs_full_groups():
    m = manager(num_pages=4, page=4)
    m.enable_prefix_cache()
    tokens = list(range(12))
    a = m.admit("a", tokens); m.extend(a, 12); m.register_full_pages(a, tokens, 12)
    m.free(a)
    b = m.admit("b", [50] * 16); m.extend(b, 16)   # takes all four pages: contents evicted
    assert m.prefix_index == {}
    m.free(b)
    c = m.admit("c", tokens)
    assert c.num_tokens == 0
    m.free(c)
    with pytest.raises(ValueError, match="keep all keys"):
        manager(windows=(None, 8)).enable_prefix_cache()


def test_chained_hash_depends_on_what_came_before():
    h = CacheManager.block_hash
    assert h([1, 2, 3, 4]) == h([1, 2, 3, 4])
    assert h([1, 2, 3, 4]) != h([1, 2, 3, 5])
    assert h([1, 2, 3, 4], h([9, 9, 9, 9])) != h([1, 2, 3, 4], h([8, 8, 8, 8]))


@pytest.mark.parametrize("seed", range(4))
def test_random_orders_with_shared_prefixes(seed):
    rnd = random.Random(seed)
    m = manager(num_pages=rnd.choice([8, 14]), page=4, slots=3)
    m.enable_prefix_cache()
    stems = [[rnd.randrange(5) for _ in range(12)] for _ in range(2)]
    live = {}
    for step in range(300):
        if rnd.random() < 0.3 and len(live) < 3:
            tokens = rnd.choice(stems) + [rnd.randrange(5) for _ in range(rnd.randrange(1, 9))]
            rc = m.admit(f"r{step}", tokens)
            assert rc.num_tokens % 4 == 0 and rc.num_tokens < len(tokens)
            live[f"r{step}"] = (rc, tokens)
        elif rnd.random() < 0.7 and live:
            rc, tokens = live[rnd.choice(sorted(live))]
            n = min(len(tokens), rc.num_tokens + rnd.choice([1, 3, 8]))
            if n > rc.num_tokens and m.can_extend(rc, n):
                m.extend(rc, n)
                m.register_full_pages(rc, tokens, n)
        elif live:
            rid = rnd.choice(sorted(live))
            m.free(live.pop(rid)[0])
        m.check()
    for rc, _ in live.values():
        m.free(rc)
    m.check()
    assert m.pools[0].num_used == 0


def test_prefix_stops_at_the_first_miss_even_if_later_blocks_would_hit():
    """The case of the reference's tests/test_block_manager.py:5-44: block 0 is a hit and in
    use, block 1 has an index entry under its hash but other tokens, blocks 2 and 3 are
    indexed and equal: one block is cached, three are new."""
    P = 4
    m = manager(num_pages=6, page=P)
    m.enable_prefix_cache()
    blocks = [[10] * P, [20] * P, [30] * P, [40] * P]
    tokens = sum(blocks, [])
    holder = m.admit("holder", tokens + [1]); m.extend(holder, 17)
    m.register_full_pages(holder, tokens + [1], 17)
    assert len(m.prefix_index) == 4
    h1 = holder.hashes[1]
    m.prefix_tokens[h1] = tuple([999] * P)         # same hash, other contents
    hit = m.match_prefix(tokens + [2])
    assert len(hit) == 1 and hit[0][1] == (holder.tables[0][0],)
    rc = m.admit("new", tokens + [2])
    assert rc.num_tokens == P                       # used: one block; new: the other three
    m.free(rc); m.free(holder)
    m.check()
