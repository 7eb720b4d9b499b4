"""The cache's bookkeeping on the host: no slot or page is lost, held twice or
freed twice; windowed groups give back pages that left the window; a step gets
all its pages or none."""
import random

import pytest

import hector_engine_amd  # noqa: F401
from hector_engine_amd.cache import CacheError, CacheFull, FreeList, GroupPages, SlotBook, blocks_for


def book(pages=16, slots=4, max_blocks=8, windows=(0,)):
    return SlotBook(slots, max_blocks, [GroupPages(pages, w, str(i)) for i, w in enumerate(windows)])


def test_free_list_lowest_first_and_double_free():
    f = FreeList(3, "thing")
    assert [f.take(), f.take(), f.take()] == [0, 1, 2]
    with pytest.raises(CacheFull):
        f.take()
    f.give_back(1)
    f.give_back(0)
    with pytest.raises(CacheError, match="not held"):
        f.give_back(0)
    assert f.take() == 0 and f.take() == 1          # reuse is deterministic: lowest first
    with pytest.raises(CacheError):
        f.give_back(7)


def test_slots_are_reused_and_pages_come_back():
    b = book()
    s0, s1 = b.acquire(), b.acquire()
    assert (s0, s1) == (0, 1)
    added = b.reserve(s0, 130)
    assert [(g, s, blk) for g, s, blk, _ in added] == [(0, 0, 0), (0, 0, 1), (0, 0, 2)]
    b.commit(s0, 130)
    b.reserve(s1, 64)
    b.commit(s1, 64)
    b.check_invariants()
    assert b.groups[0].pool.available == 16 - 4
    cleared = b.release(s0)
    assert len(cleared) == 3 and b.groups[0].pool.available == 15
    assert b.acquire() == 0                            # the freed slot is handed out again
    with pytest.raises(CacheError):
        b.release(3)                                   # never acquired
    b.check_invariants()


def test_reserve_is_all_or_nothing():
    b = book(pages=4, windows=(0, 0))
    s = b.acquire()
    b.reserve(s, 200)                                  # 4 pages in each group... exactly fits
    t = b.acquire()
    with pytest.raises(CacheFull):
        b.reserve(t, 1)
    assert b.groups[0].table[t] == [] and b.groups[1].table[t] == []
    b.check_invariants()
    with pytest.raises(CacheFull, match="longest sequence"):
        _too_long()


def _too_long():
    b = book(pages=64, max_blocks=2)
    b.reserve(b.acquire(), 129)


def test_cannot_shrink():
    b = book()
    s = b.acquire()
    b.reserve(s, 10)
    b.commit(s, 10)
    with pytest.raises(CacheError, match="shrink"):
        b.reserve(s, 5)


@pytest.mark.parametrize("window", [1, 8, 64, 70, 129])
def test_window_group_frees_exactly_the_dead_blocks(window):
    b = book(pages=32, max_blocks=16, windows=(0, window))
    s = b.acquire()
    for new_len in (3, 64, 65, 130, 200, 512, 513, 700):
        b.reserve(s, new_len)
        b.commit(s, new_len)
        b.check_invariants()
        full, win = b.groups[0].table[s], b.groups[1].table[s]
        assert all(p >= 0 for p in full) and len(full) == blocks_for(new_len)
        for blk, page in enumerate(win):
            last_pos = 64 * blk + 63
            # a later query at p >= new_len sees keys > p - window >= new_len - window
            dead = last_pos <= new_len - window
            assert (page < 0) == dead, (new_len, blk)
    b.release(s)
    assert b.groups[1].pool.available == 32 and b.groups[0].pool.available == 32


def test_random_traffic_keeps_every_invariant():
    rng = random.Random(0)
    b = book(pages=40, slots=6, max_blocks=12, windows=(0, 70))
    live = {}
    for _ in range(3000):
        op = rng.random()
        if op < 0.25 and len(live) < 6:
            live[b.acquire()] = 0
        elif op < 0.45 and live:
            s = rng.choice(list(live))
            b.release(s)
            del live[s]
        elif live:
            s = rng.choice(list(live))
            new = live[s] + rng.choice([1, 1, 1, 5, 64, 100])
            try:
                b.reserve(s, new)
                b.commit(s, new)
                live[s] = new
            except CacheFull:
                pass
        b.check_invariants()
        assert set(b.length) == set(live) and all(b.length[s] == n for s, n in live.items())
    for s in list(live):
        b.release(s)
    assert all(g.pool.available == 40 for g in b.groups) and b.slots.available == 6


def test_truncate_gives_back_whole_pages_beyond_the_new_length():
    b = book(pages=16, windows=(0, 0))
    s = b.acquire()
    b.reserve(s, 300)
    b.commit(s, 300)
    assert b.groups[0].pool.available == 16 - 5
    cleared = b.truncate(s, 130)                      # 130 tokens lie in 3 pages
    assert sorted(cleared) == [(0, s, 3), (0, s, 4), (1, s, 3), (1, s, 4)]
    assert b.length[s] == 130 and b.groups[0].pool.available == 16 - 3
    b.check_invariants()
    assert b.truncate(s, 129) == [] and b.length[s] == 129      # same pages, shorter
    b.reserve(s, 200)                                 # grows again into pages handed out anew
    b.commit(s, 200)
    b.check_invariants()
    b.truncate(s, 0)
    assert b.groups[0].table[s] == [] and b.groups[0].pool.available == 16
    with pytest.raises(CacheError, match="truncate"):
        b.truncate(s, 1)                              # longer than the slot
    with pytest.raises(CacheError):
        b.truncate(3, 0)                              # never acquired
    b.release(s)
    b.check_invariants()


def test_truncate_of_a_windowed_group_needs_the_window_it_gave_back():
    b = book(pages=32, max_blocks=16, windows=(0, 70))
    s = b.acquire()
    b.reserve(s, 400)
    b.commit(s, 400)               # positions <= 330 left the window: blocks 0..4 were given back
    assert [p < 0 for p in b.groups[1].table[s]] == [True] * 5 + [False] * 2
    b.truncate(s, 390)             # a query at 390 reads keys > 320: block 5 (320..383) is still there
    assert b.length[s] == 390
    before = (list(b.groups[0].table[s]), list(b.groups[1].table[s]), b.groups[1].pool.available)
    with pytest.raises(CacheError, match="window"):
        b.truncate(s, 380)         # a query at 380 reads keys > 310: block 4 (256..319) is gone
    assert before == (list(b.groups[0].table[s]), list(b.groups[1].table[s]), b.groups[1].pool.available)
    assert b.length[s] == 390      # nothing was changed
    b.check_invariants()


def test_random_traffic_with_truncation_keeps_every_invariant():
    rng = random.Random(1)
    b = book(pages=40, slots=5, max_blocks=12, windows=(0, 100))
    live = {}
    for _ in range(3000):
        op = rng.random()
        if op < 0.2 and len(live) < 5:
            live[b.acquire()] = 0
        elif op < 0.3 and live:
            s = rng.choice(list(live))
            b.release(s)
            del live[s]
        elif op < 0.5 and live:
            s = rng.choice(list(live))
            new = rng.randint(0, live[s])
            try:
                b.truncate(s, new)
                live[s] = new
            except CacheError:
                pass                                   # the window's pages were gone: nothing changed
        elif live:
            s = rng.choice(list(live))
            new = live[s] + rng.choice([1, 1, 5, 64, 100])
            try:
                b.reserve(s, new)
                b.commit(s, new)
                live[s] = new
            except CacheFull:
                pass
        b.check_invariants()
        assert all(b.length[s] == n for s, n in live.items())
        for s, n in live.items():                      # every position a next query reads has a page
            for g in b.groups:
                first = max(0, n - g.window + 1) if g.window else 0
                assert len(g.table[s]) == blocks_for(n)
                assert all(g.table[s][blk] >= 0 for blk in range(first // 64, blocks_for(n)))
    for s in list(live):
        b.release(s)
    assert all(g.pool.available == 40 for g in b.groups)


def test_the_host_copy_of_the_page_tables_follows_the_device_tables():
    """The cache keeps its page tables twice, for the kernels and for the step's metadata: after
    every kind of traffic (growth, a window that moves on, truncation, release, a slot used again)
    both say the same, in a group that keeps all keys and in one that keeps a window."""
    import numpy as np
    import torch
    from hector_engine_amd.cache.paged import PagedCache, RunPlan
    from hector_engine_amd.parts.base import KVNeed
    plans = [RunPlan(KVNeed(2, 16), None), RunPlan(KVNeed(2, 16, window=100), None), RunPlan(None, 0)]
    cache = PagedCache(plans, max_tokens=64 * 24, max_slots=4, max_seq_len=64 * 8, dtype=torch.float32,
                       device="cpu")
    rng = random.Random(5)
    held: dict[int, int] = {}

    def check():
        for g in cache.groups:
            assert np.array_equal(g.host_table, g.page_table.numpy())
        slots = sorted(held)
        out = np.full((len(cache.groups), len(slots) + 2, cache.max_blocks), 7, dtype=np.int32)
        cache.rows_of_tables(slots, out)
        for gi, g in enumerate(cache.groups):
            assert np.array_equal(out[gi, :len(slots)], g.page_table.numpy()[slots])
            assert (out[gi, len(slots):] == 7).all()

    for _ in range(300):
        move = rng.random()
        try:
            if move < 0.2 and len(held) < cache.max_slots:
                held[cache.acquire()] = 0
            elif move < 0.75 and held:
                s = rng.choice(sorted(held))
                n = held[s] + rng.choice([1, 1, 1, 63, 64, 130])
                cache.reserve([(s, n)])
                cache.commit([(s, n)])
                held[s] = n
            elif move < 0.85 and held:
                s = rng.choice(sorted(held))
                n = rng.randrange(held[s] + 1)
                cache.truncate(s, n)
                held[s] = n
            elif held:
                s = rng.choice(sorted(held))
                cache.release(s)
                del held[s]
        except (CacheFull, CacheError):
            pass
        check()
    assert any((g.host_table >= 0).any() for g in cache.groups)
