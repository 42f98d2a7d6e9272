"""Slots and pages: nothing lost, held twice or freed twice (no GPU)."""
import random

import pytest

from edge_infer_amd.cache import (PAGE_TOKENS, CacheFull, PagePool, SequencePages, SlotTable,
                                  pages_for)


def test_pages_for():
    assert [pages_for(n) for n in (0, 1, 64, 65, 128)] == [0, 1, 1, 2, 2]
    assert PAGE_TOKENS == 64


def test_page_pool_rules():
    pool = PagePool(5)
    a = pool.alloc(3)
    assert a == [0, 1, 2] and pool.n_free == 2
    with pytest.raises(CacheFull):
        pool.alloc(3)
    assert pool.n_free == 2            # a refused request changes nothing
    pool.free([1])
    with pytest.raises(RuntimeError, match="twice"):
        pool.free([1])
    with pytest.raises(RuntimeError, match="twice"):
        pool.free([0, 0])
    with pytest.raises(ValueError):
        pool.free([9])
    assert pool.n_free == 3
    b = pool.alloc(3)
    assert sorted(b) == [1, 3, 4] and not set(b) & {0, 2}
    pool.check()


def test_slot_table_rules():
    table = SlotTable(3)
    s = [table.acquire() for _ in range(3)]
    assert sorted(s) == [0, 1, 2]
    with pytest.raises(CacheFull):
        table.acquire()
    table.release(1)
    with pytest.raises(RuntimeError, match="twice"):
        table.release(1)
    assert table.acquire() == 1         # the slot is used again
    assert table.live_slots() == [0, 1, 2]
    table.check()


def test_random_traffic_keeps_every_page_accounted():
    rng = random.Random(3)
    pool = PagePool(40)
    slots = SlotTable(6)
    pages = SequencePages(pool, 6)
    live = {}
    for _ in range(3000):
        action = rng.random()
        if action < 0.25 and slots.n_free:
            slot = slots.acquire()
            pages.open(slot)
            live[slot] = 0
        elif action < 0.8 and live:
            slot = rng.choice(list(live))
            new_length = live[slot] + rng.randint(1, 200)
            need = pages.pages_needed(slot, new_length)
            if need > pool.n_free:
                with pytest.raises(CacheFull):
                    pages.grow(slot, new_length)
            else:
                pages.grow(slot, new_length)
                live[slot] = new_length
                assert len(pages.row(slot)) == pages_for(new_length)
        elif live:
            slot = rng.choice(list(live))
            pages.close(slot)
            slots.release(slot)
            del live[slot]
        pool.check()
        slots.check()
        held = [p for s in live for p in pages.row(s)]
        assert len(held) == len(set(held)) == pool.n_pages - pool.n_free
    for slot in list(live):
        pages.close(slot)
        slots.release(slot)
    assert pool.n_free == 40 and slots.n_free == 6


def test_window_group_gives_dead_pages_back():
    pool = PagePool(8)
    pages = SequencePages(pool, 1, window=70)
    pages.open(0)
    pages.grow(0, 200)                  # pages 0..3
    assert pool.n_free == 4
    pages.trim(0, 200)                  # next query at 200 sees keys 131..200: pages 0, 1 dead
    assert list(pages.row(0)) == [-1, -1, 2, 3] and pool.n_free == 6
    pages.trim(0, 200)                  # trimming again frees nothing twice
    assert pool.n_free == 6
    pages.grow(0, 260)                  # one more page; logical index 4
    assert len(pages.row(0)) == 5 and pages.row(0)[4] in (0, 1, 4)
    pages.close(0)
    assert pool.n_free == 8
    pool.check()
    full = SequencePages(PagePool(4), 1, window=None)
    full.open(0)
    full.grow(0, 256)
    full.trim(0, 256)
    assert list(full.row(0)) == [0, 1, 2, 3]
