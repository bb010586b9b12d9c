"""Cache manager: block tables, groups, window release, state slots; no page is
lost, held twice or freed twice under random orders of requests (no GPU)."""
import random

import pytest

from servelab_amd.cache import CacheManager, PageAllocator, RELEASED, SlotAllocator
from servelab_amd.parts import PagedKVSpec, StateSpec

FULL = PagedKVSpec(2, 16, None)
WIN = PagedKVSpec(2, 16, 16)


def test_reference_vectors():
    # tests/test_block_manager.py:10-22 of the reference: 8 tokens at page size 4
    m = CacheManager({0: FULL}, num_pages=16, page_size=4)
    assert m.open("s1")
    assert m.grow("s1", 8)
    got = list(m.block_table(0, "s1"))
    assert len(got) == 2
    assert m.grow("s1", 9) and len(m.block_table(0, "s1")) == 3      # one more token: a new page
    assert m.slot(0, "s1", 0) == got[0] * 4 + 0
    assert m.slot(0, "s1", 5) == got[1] * 4 + 1
    m.close("s1")
    assert m.num_free_pages() == 16                                   # :80-86
    m.check()


def test_fifo_reuse_and_all_or_nothing():
    m = CacheManager({0: FULL, 1: FULL, 2: WIN}, num_pages=4, page_size=16)
    assert len(m.page_groups) == 2 and m.page_groups[0].streams == [0, 1]
    m.open("a")
    assert m.grow("a", 40)                   # 3 pages in both groups
    m.open("b")
    assert not m.grow("b", 17)               # needs 2, 1 free: nothing is taken
    assert m.block_table(0, "b") == [] and m.block_table(1, "b") == []
    assert m.grow("b", 16)
    first = list(m.block_table(0, "a"))
    m.close("a")
    m.open("c")
    assert m.grow("c", 48)
    assert m.block_table(0, "c") == first    # freed pages come back in order
    m.check()
    assert not m.can_ever_hold(65) and m.can_ever_hold(64)


def test_grow_twice_is_harmless():
    m = CacheManager({0: FULL}, num_pages=8, page_size=16)
    m.open("a")
    assert m.grow("a", 20) and m.grow("a", 20) and m.grow("a", 5)
    assert len(m.block_table(0, "a")) == 2


def test_window_pages_are_given_back():
    m = CacheManager({0: FULL, 1: WIN}, num_pages=16, page_size=16)
    m.open("a")
    m.grow("a", 100)
    m.commit("a", 100)
    full, win = m.block_table(0, "a"), m.block_table(1, "a")
    assert RELEASED not in full and len(full) == 7
    # keys r <= 100 - 16 = 84 are dead: pages 0..4 hold tokens 0..79, page 5 holds 80..95
    assert win[:5] == [RELEASED] * 5 and RELEASED not in win[5:]
    assert m.page_groups[1].allocator.num_used == 2
    m.grow("a", 101)
    m.commit("a", 101)                                              # 101 - 16 = 85: still page 5
    assert m.block_table(1, "a")[5] != RELEASED
    m.grow("a", 112)
    m.commit("a", 112)                                              # 96 > 95: page 5 goes
    assert m.block_table(1, "a")[5] == RELEASED
    with pytest.raises(AssertionError):
        m.slot(1, "a", 3)
    m.check()
    m.close("a")
    m.check()
    assert m.num_free_pages() == 16


def test_state_slots():
    m = CacheManager({0: FULL, 1: StateSpec((4, 8))}, num_pages=8, page_size=16, num_state_slots=2)
    assert len(m.state_groups) == 1 and m.stream_group[1][0] == "state"
    assert m.open("a") and m.open("b")
    assert {m.state_slot("a"), m.state_slot("b")} == {0, 1}
    assert not m.open("c")                       # no slot: nothing opened
    assert not m.is_open("c")
    m.close("a")
    assert m.open("c") and m.state_slot("c") == 0
    m.check()
    # an architecture without state still has the slot array
    q = CacheManager({0: FULL}, num_pages=8, page_size=16, num_state_slots=4)
    assert q.state_groups == [] and q.state_slots.num_slots == 4


def test_double_free_and_double_hold_are_errors():
    a = PageAllocator(4)
    pages = a.take(2)
    a.give(pages)
    with pytest.raises(AssertionError):
        a.give(pages[:1])
    s = SlotAllocator(2)
    s.take("x")
    with pytest.raises(AssertionError):
        s.take("x")


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_conserve_pages(seed):
    rng = random.Random(seed)
    m = CacheManager({0: FULL, 1: FULL, 2: WIN, 3: PagedKVSpec(1, 32, 40)}, num_pages=24,
                     page_size=16, num_state_slots=6)
    live = {}
    for step in range(600):
        action = rng.random()
        if action < 0.25 and len(live) < 6:
            rid = f"r{step}"
            assert m.open(rid)
            live[rid] = 0
        elif action < 0.8 and live:
            rid = rng.choice(list(live))
            total = live[rid] + rng.choice([1, 1, 1, 2, 7, 24, 50])
            before = [g.allocator.num_free for g in m.page_groups]
            if m.grow(rid, total):
                m.commit(rid, total)
                live[rid] = total
            else:
                assert before == [g.allocator.num_free for g in m.page_groups]
        elif live:
            rid = rng.choice(list(live))
            m.close(rid)
            del live[rid]
        m.check()
        for g in m.page_groups:                 # every live token of every group has a page
            for rid, n in live.items():
                lo = 0 if g.window is None else max(0, n - g.window + 1)
                for tok in (lo, n - 1):
                    if n:
                        assert g.tables[rid][tok // 16] != RELEASED
    for rid in list(live):
        m.close(rid)
    m.check()
    assert all(g.allocator.num_free == 24 for g in m.page_groups)
