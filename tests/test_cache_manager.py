"""The cache manager's book-keeping (CPU): no page lost, held twice or freed twice, under
random orders of requests; windows give pages back; failures take nothing."""
import random

import pytest

from tuff_amd.cache.manager import (FREED, CacheError, CacheLayout, CacheManager, OutOfPages, OutOfSlots,
                                    PagePool)
from tuff_amd.parts.base import FixedState, PagedKV


def layout(windows=(None,), states=1):
    specs = {}
    for i, w in enumerate(windows):
        specs[i] = PagedKV(2, 16, w)
    for j in range(states):
        specs[100 + j] = FixedState((2, 8))
    return CacheLayout.from_specs(specs)


def test_page_pool_hands_out_each_page_once_and_refuses_double_free():
    pool = PagePool(5)
    a = pool.alloc(3)
    b = pool.alloc(2)
    assert sorted(a + b) == [0, 1, 2, 3, 4] and pool.num_free == 0
    with pytest.raises(OutOfPages):
        pool.alloc(1)
    pool.free(a)
    with pytest.raises(CacheError, match="not held"):
        pool.free([a[0]])
    with pytest.raises(CacheError, match="not held"):
        pool.free([99])
    again = pool.alloc(3)
    assert sorted(again) == sorted(a)                      # freed pages are used again
    assert again[0] == a[-1]                               # last freed, first used


def test_groups_by_window_and_shared_page_numbering():
    lay = CacheLayout.from_specs({0: PagedKV(2, 16), 1: FixedState((2, 8)), 2: PagedKV(4, 8), 3: PagedKV(2, 16, 32),
                                  4: PagedKV(1, 64, 32), 5: None})
    assert lay.group_windows == [None, 32]
    assert lay.group_of_entry == {0: 0, 2: 0, 3: 1, 4: 1}
    assert lay.bytes_per_token(2) == 2 * 2 * (2 * 16 + 4 * 8 + 2 * 16 + 64)
    assert lay.state_bytes_per_request() == 2 * 8 * 4
    # values of a width of their own: a token costs keys + values, not twice the keys
    assert PagedKV(2, 16).v_dim == 16 and PagedKV(2, 16, None, 40).v_dim == 40
    assert CacheLayout.from_specs({0: PagedKV(2, 16, value_dim=40)}).bytes_per_token(2) == 2 * 2 * (16 + 40)
    with pytest.raises(CacheError, match="unknown cache declaration"):
        CacheLayout.from_specs({0: "ring buffer"})


def test_extend_release_and_lookup():
    m = CacheManager(layout(), page_size=4, num_pages=6, num_slots=2)
    s = m.admit("a")
    assert s == 0 and m.length("a") == 0 and m.block_table("a", 0) == []
    m.extend("a", 5)
    assert len(m.block_table("a", 0)) == 2 and m.length("a") == 5
    m.extend("a", 3)                                       # fills the second page exactly
    assert len(m.block_table("a", 0)) == 2
    m.extend("a", 1)
    t = m.block_table("a", 0)
    assert len(t) == 3
    assert m.slot_of_position("a", 0, 8) == t[2] * 4 and m.slot_of_position("a", 0, 7) == t[1] * 4 + 3
    m.check()
    m.admit("b")
    with pytest.raises(OutOfSlots):
        m.admit("c")
    with pytest.raises(CacheError, match="already live"):
        m.admit("a")
    with pytest.raises(OutOfPages):
        m.extend("b", 13)                                  # 4 pages wanted, 3 free
    assert m.length("b") == 0 and m.block_table("b", 0) == []          # nothing was taken
    assert not m.can_extend("b", 13) and m.can_extend("b", 12)
    m.extend("b", 12)
    m.check()
    m.release("a")
    assert m.groups[0].pool.num_free == 3 and m.free_slots == 1
    with pytest.raises(CacheError, match="holds no cache"):
        m.release("a")
    m.release("b")
    m.check()
    assert m.groups[0].pool.num_free == 6 and m.free_slots == 2


def test_truncate_takes_back_an_extend():
    m = CacheManager(layout(), page_size=4, num_pages=4, num_slots=1)
    m.admit("a")
    m.extend("a", 6)
    m.extend("a", 7)
    m.truncate("a", 6)
    assert m.length("a") == 6 and len(m.block_table("a", 0)) == 2 and m.groups[0].pool.num_free == 2
    m.check()
    with pytest.raises(CacheError):
        m.truncate("a", 7)


def test_window_gives_pages_back_once_passed():
    m = CacheManager(layout(windows=(None, 6)), page_size=4, num_pages=[16, 3], num_slots=1)
    m.admit("a")
    full, win = m.groups[0].pool, m.groups[1].pool
    for step in range(40):
        m.extend("a", 1)
        m.check()
        L = m.length("a")
        # every key the newest token reads is still there: positions L-6 .. L-1
        for pos in range(max(0, L - 6), L):
            m.slot_of_position("a", 1, pos)
        assert len(m.block_table("a", 0)) == -(-L // 4)
        assert win.num_pages - win.num_free <= 3
    assert m.block_table("a", 1)[0] == FREED
    with pytest.raises(CacheError, match="given back"):
        m.slot_of_position("a", 1, 0)
    assert win.allocations > win.num_pages                  # pages went round
    assert full.num_pages - full.num_free == 10
    m.release("a")
    m.check()
    assert win.num_free == 3 and full.num_free == 16


def test_window_portion_keeps_what_its_first_token_reads():
    """A portion of 10 tokens after 9: its first token (position 9) reads 4..9 with window 6, so the
    block of positions 4..7 must survive the extend although the last token no longer needs it."""
    m = CacheManager(layout(windows=(6,)), page_size=4, num_pages=8, num_slots=1)
    m.admit("a")
    m.extend("a", 9)
    m.extend("a", 10)
    t = m.block_table("a", 0)
    assert t[0] == FREED and t[1] != FREED
    m.extend("a", 1)                                        # now position 19 reads 14..19
    t = m.block_table("a", 0)
    assert t[:3] == [FREED] * 3 and t[3] != FREED
    m.check()


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_lose_nothing(seed):
    rng = random.Random(seed)
    ps = rng.choice([1, 4, 16])
    m = CacheManager(layout(windows=(None, rng.choice([5, 40])), states=2), page_size=ps,
                     num_pages=[rng.randrange(8, 30), rng.randrange(4, 12)], num_slots=4)
    live, next_id = {}, 0
    for _ in range(600):
        action = rng.random()
        if action < 0.15 and m.free_slots:
            m.admit(next_id)
            live[next_id] = 0
            next_id += 1
        elif action < 0.8 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 3, 7, 20])
            ok = m.can_extend(rid, n)
            before = [list(m.block_table(rid, g)) for g in range(2)]
            try:
                m.extend(rid, n)
                assert ok
                live[rid] += n
            except OutOfPages:
                assert not ok
                # nothing but window releases happened
                for g in range(2):
                    after = m.block_table(rid, g)
                    assert len(after) == len(before[g])
                    assert all(a == b or a == FREED for a, b in zip(after, before[g]))
            assert m.length(rid) == live[rid]
        elif action < 0.9 and live:
            rid = rng.choice(list(live))
            cut = rng.randrange(0, live[rid] + 1)
            if cut >= live[rid] - 3:                        # only the latest extend is ever taken back
                m.truncate(rid, cut)
                live[rid] = cut
        elif live:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
        m.check()
    for rid in list(live):
        m.release(rid)
    m.check()
    assert all(g.pool.num_free == g.pool.num_pages for g in m.groups) and m.free_slots == 4
