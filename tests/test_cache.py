"""The cache's bookkeeping: pages and slots are never lost, held twice or freed twice (no GPU;
storage lives on the CPU here)."""
import random

import pytest
import torch

from picolm_amd.cache import (Cache, CacheError, CacheFull, CacheSpec, KVGroupSpec, PagedGroupBook, PagePool, SlotTable,
                              StateGroupSpec, pages_for, window_ring_pages)


def test_page_pool():
    p = PagePool(5)
    a = p.take(3)
    assert sorted(a) == [0, 1, 2] and p.n_free == 2
    with pytest.raises(CacheFull):
        p.take(3)
    assert p.n_free == 2                       # a refused request takes nothing
    p.give(a[:1])
    with pytest.raises(CacheError, match="twice"):
        p.give(a[:1])
    with pytest.raises(CacheError, match="not of this pool"):
        p.give([9])
    b = p.take(3)
    assert len(set(b) | set(a[1:])) == 5       # nothing handed out twice


def test_slot_table():
    s = SlotTable(2)
    a, b = s.alloc(), s.alloc()
    assert {a, b} == {0, 1}
    with pytest.raises(CacheFull):
        s.alloc()
    s.free(a)
    with pytest.raises(CacheError, match="twice"):
        s.free(a)
    with pytest.raises(CacheError, match="does not exist"):
        s.free(7)
    assert s.alloc() == a and s.live_slots() == [0, 1]


def test_window_ring():
    # a ring holds a window and one chunk of new tokens, wherever they start in a page
    assert window_ring_pages(1, 64) == 2 and window_ring_pages(65, 64) == 3 and window_ring_pages(66, 64) == 4
    assert window_ring_pages(100) == pages_for(99 + 256) + 1 == 7
    book = PagedGroupBook(10, 2, ring_pages=3)
    assert [j for j, _ in book.grow(0, 1000)] == [0, 1, 2]     # never more than the ring
    assert book.grow(0, 5000) == []
    book.release(0)
    assert book.pool.n_free == 10


def make_cache(max_tokens=64 * 8, n_slots=4, max_seq_len=64 * 5):
    spec = CacheSpec([KVGroupSpec(2, 2, 16), KVGroupSpec(1, 1, 32, window=100)],
                     [StateGroupSpec(3, (4, 2), torch.float32)])
    return Cache(spec, max_tokens, max_seq_len, torch.float32, "cpu", n_slots)


def test_cache_shapes_and_groups():
    c = make_cache()
    full, win = c.kv
    assert tuple(full.k.shape) == (2, 8, 2, 64, 16) and tuple(full.v.shape) == (2, 8, 2, 16, 64)
    assert win.ring_pages == 5 and tuple(win.k.shape) == (1, 8, 1, 64, 32)     # capped by a sequence's 5 pages
    assert full.k.data_ptr() != win.k.data_ptr()
    assert tuple(c.state[0].shape) == (3, 4, 4, 2)
    assert c.max_seq_len == 320 and c.max_pages == 5


def test_values_of_another_size_than_keys():
    from picolm_amd.parts import KVRequest
    assert KVRequest(2, 16, 0, 16) == KVRequest(2, 16) and KVRequest(2, 16).value_dim == 16
    assert KVRequest(2, 16, 0, 24) != KVRequest(2, 16) and KVRequest(2, 16, 0, 24).value_dim == 24
    c = Cache(CacheSpec([KVGroupSpec(1, 2, 16, 0, 24)], []), 128, 128, torch.float32, "cpu", 2)
    (g,) = c.kv
    assert tuple(g.k.shape) == (1, 2, 2, 64, 16) and tuple(g.v.shape) == (1, 2, 2, 24, 64)
    assert g.bytes() == 4 * 2 * 2 * 64 * (16 + 24) == c.bytes()


def test_reserve_is_all_or_nothing_and_lengths_are_per_slot():
    c = make_cache()
    a, b = c.alloc_slot(), c.alloc_slot()
    c.reserve(a, 130)
    assert len(c.kv[0].book.pages[a]) == 3 and len(c.kv[1].book.pages[a]) == 3
    c.set_length(a, 130)
    assert c.length(a) == 130 and c.length(b) == 0
    with pytest.raises(CacheFull):
        c.reserve(b, 64 * 6)                    # longer than a sequence may get
    with pytest.raises(CacheFull):
        c.reserve_many([a, b], [300, 300])      # 5 + 5 pages > 8
    assert len(c.kv[0].book.pages[a]) == 3 and len(c.kv[0].book.pages[b]) == 0
    c.reserve_many([a, b], [200, 250])
    assert c.kv[0].book.pool.n_free == 0
    tab = c.kv[0].table_host
    held = [int(tab[a, j]) for j in range(4)] + [int(tab[b, j]) for j in range(4)]
    assert sorted(held) == list(range(8))
    c.flush()
    assert torch.equal(c.kv[0].table, tab) and not c.kv[0].dirty
    with pytest.raises(CacheError, match="not live"):
        c.reserve(3, 10)


def test_slots_are_given_back_and_used_again():
    c = make_cache()
    a = c.alloc_slot()
    c.reserve(a, 300)
    c.state[0][:, a] = 7.0
    c.free_slot(a)
    assert c.kv[0].book.pool.n_free == 8 and c.kv[1].book.pool.n_free == 8
    with pytest.raises(CacheError, match="twice"):
        c.free_slot(a)
    assert c.kv[0].book.pool.n_free == 8       # the refused free moved no page
    a2 = c.alloc_slot()
    assert a2 == a and c.length(a2) == 0
    assert float(c.state[0][:, a2].abs().sum()) == 0.0          # state starts at zero in a reused slot


def test_random_walk_keeps_the_books_balanced():
    rnd = random.Random(0)
    c = make_cache(max_tokens=64 * 20, n_slots=6, max_seq_len=64 * 8)
    live = {}
    for _ in range(2000):
        op = rnd.random()
        if op < 0.3 and len(live) < 6:
            live[c.alloc_slot()] = 0
        elif op < 0.8 and live:
            s = rnd.choice(list(live))
            n = min(live[s] + rnd.randint(1, 90), c.max_seq_len)
            try:
                c.reserve(s, n)
                c.set_length(s, n)
                live[s] = n
            except CacheFull:
                pass
        elif live:
            s = rnd.choice(list(live))
            c.free_slot(s)
            del live[s]
        for g in c.kv:
            held = [p for s in range(c.n_slots) for p in g.book.pages[s]]
            assert len(held) == len(set(held))                                  # no page held twice
            assert len(held) + g.book.pool.n_free == g.book.pool.n_pages        # none lost
            for s in range(c.n_slots):
                want = g.book.need(live[s]) if s in live else 0
                assert len(g.book.pages[s]) == want
        assert sorted(live) == c.slots.live_slots()
        assert c.slots.n_free + len(live) == c.n_slots


def test_a_refused_batch_leaves_the_books_as_they_were():
    c = make_cache(max_tokens=64 * 20, n_slots=4, max_seq_len=64 * 4)
    a, b = c.alloc_slot(), c.alloc_slot()
    free = [g.book.pool.n_free for g in c.kv]
    with pytest.raises(CacheFull):
        c.reserve_many([a, b], [100, 64 * 4 + 1])          # the last sequence is too long: nothing may grow
    assert [g.book.pool.n_free for g in c.kv] == free
    assert all(len(g.book.pages[a]) == 0 for g in c.kv)
    c.free_slot(b)
    with pytest.raises(CacheError, match="not live"):
        c.reserve_many([a, b], [100, 10])                  # a dead slot behind a good one
    assert [g.book.pool.n_free for g in c.kv] == free
    c.reserve_many([a], [100])
    assert all(len(g.book.pages[a]) == g.book.need(100) for g in c.kv)
