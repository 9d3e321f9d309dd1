"""The page and slot manager: no page lost, held twice or freed twice, under random
orders of requests; first-in first-out reuse; windows; state slots."""
import random

import pytest

from yalis_amd.cache.manager import CacheError, GroupShape, PageManager


def test_reserve_release_and_fifo_reuse():
    m = PageManager(16, [GroupShape(6)], num_slots=2)
    assert m.admit(10) == 0 and m.admit(11) == 1 and m.admit(12) is None, "slots smallest first, then none"
    assert m.reserve(10, 17)  # two pages
    assert m.block_table(10, 0).tolist() == [0, 1]
    assert m.reserve(10, 32) and m.block_table(10, 0).tolist() == [0, 1], "no page until a boundary is crossed"
    assert m.reserve(10, 33) and m.block_table(10, 0).tolist() == [0, 1, 2]
    assert m.reserve(11, 40) and m.block_table(11, 0).tolist() == [3, 4, 5]
    assert m.free_pages(0) == 0
    assert not m.reserve(10, 49), "the pool is empty: refused without an exception"
    assert m.block_table(10, 0).tolist() == [0, 1, 2], "a refused reservation changes nothing"
    m.audit()
    assert m.release(10) == 3
    assert m.free_list(0) == [0, 1, 2], "pages go to the back of the free list in table order"
    assert m.admit(12) == 0, "the freed slot is the smallest again"
    assert m.reserve(12, 20) and m.block_table(12, 0).tolist() == [0, 1], "and are taken from the front"
    m.audit()
    with pytest.raises(CacheError, match="already live"):
        m.admit(12)
    with pytest.raises(CacheError, match="unknown request"):
        m.release(99)
    with pytest.raises(CacheError, match="unknown request"):
        m.reserve(10, 5)  # released above: cannot be freed or grown twice


def test_groups_are_all_or_nothing():
    m = PageManager(16, [GroupShape(4), GroupShape(2)], num_slots=4)
    m.admit(1)
    assert m.pages_needed(1, 40) == [3, 3]
    assert not m.reserve(1, 40), "the second group has two pages only"
    assert m.free_pages(0) == 4 and m.free_pages(1) == 2
    assert m.reserve(1, 32)
    assert m.block_tables(1)[0].tolist() == [0, 1] and m.block_tables(1)[1].tolist() == [0, 1]
    m.audit()


def test_window_gives_pages_back():
    m = PageManager(16, [GroupShape(8), GroupShape(8, window=20)], num_slots=1)
    m.admit(5)
    assert m.reserve(5, 70)  # five pages in both groups
    assert m.advance(5, 19) == 0
    # with 35 tokens cached the next query (position 35) reads keys 16..35: page 0 (keys 0..15) is dead
    assert m.advance(5, 34) == 0 and m.advance(5, 35) == 1
    assert m.block_table(5, 1).tolist() == [-1, 1, 2, 3, 4]
    assert m.block_table(5, 0).tolist() == [0, 1, 2, 3, 4], "the unwindowed group keeps everything"
    assert m.advance(5, 70) == 2  # keys <= 50 are dead: pages 0..2
    assert m.block_table(5, 1).tolist() == [-1, -1, -1, 3, 4]
    assert m.free_list(1) == [5, 6, 7, 0, 1, 2]
    assert m.reserve(5, 100) and m.block_table(5, 1).tolist()[5:] == [5, 6], "growth takes new pages at the end"
    m.audit()
    assert m.release(5) == 7 + 4
    m.audit()
    assert m.free_pages(0) == 8 and m.free_pages(1) == 8


@pytest.mark.parametrize("seed", range(5))
def test_random_orders_keep_the_books(seed):
    rng = random.Random(seed)
    page, n_pages, n_slots = 16, 24, 5
    m = PageManager(page, [GroupShape(n_pages), GroupShape(n_pages, window=40)], n_slots)
    live = {}
    next_id = 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and len(live) < n_slots:
            assert m.admit(next_id) is not None
            live[next_id] = 0
            next_id += 1
        elif op < 0.8 and live:
            r = rng.choice(list(live))
            grow = rng.choice([1, 1, 1, 2, 7, 16, 33, 50])
            before = (m.free_pages(0), m.free_pages(1), m.block_tables(r))
            if m.reserve(r, live[r] + grow):
                live[r] += grow
                m.advance(r, live[r])
                assert len(m.block_table(r, 0)) == -(-live[r] // page)
            else:
                after = (m.free_pages(0), m.free_pages(1), m.block_tables(r))
                assert before[:2] == after[:2] and all((a == b).all() for a, b in zip(before[2], after[2]))
        elif live:
            r = rng.choice(list(live))
            m.release(r)
            del live[r]
        m.audit()
        held0 = sum(len(m.block_table(r, 0)) for r in live)
        assert held0 + m.free_pages(0) == n_pages
        held1 = sum(int((m.block_table(r, 1) >= 0).sum()) for r in live)
        assert held1 + m.free_pages(1) == n_pages
        assert m.live_requests() == len(live) and m.free_slots() == n_slots - len(live)
        slots = [m.slot(r) for r in live]
        assert len(set(slots)) == len(slots)
    for r in list(live):
        m.release(r)
    m.audit()
    assert m.free_pages(0) == n_pages and m.free_pages(1) == n_pages and m.free_slots() == n_slots
