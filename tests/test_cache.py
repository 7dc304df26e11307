"""The cache's bookkeeping (csrc/engine.hip), without a GPU: pages and slots are never lost, held
twice or freed twice; a group that keeps a window of keys holds a ring of pages per slot and never
more; a step's reservation is all or nothing over every group."""
import random

import pytest

from host_engine import host_engine
from picolm_amd.cache import CacheError, CacheFull, pages_for, window_ring_pages


def test_window_ring():
    # a ring holds a window and one chunk of new tokens, wherever they start in a page
    assert window_ring_pages(1, 64) == 2 and window_ring_pages(65, 64) == 3 and window_ring_pages(66, 64) == 4
    assert window_ring_pages(100) == pages_for(99 + 256) + 1 == 7


def test_groups_have_storage_of_their_own():
    e = host_engine(max_tokens=64 * 40, max_seq_len=64 * 16, n_slots=2, layers=3, windows=(0, 100))
    assert e.kv_pages(0) == 32 and e.kv_pages(1) == 14              # every page a slot could hold; two rings of seven
    a = e.slot_alloc()
    e.step([a], [[1] * 200])
    assert len(e.slot_pages(0, a)) == 4 and len(e.slot_pages(1, a)) == 4
    e.step([a], [[1] * 256])
    e.step([a], [[1] * 256])
    assert len(e.slot_pages(0, a)) == pages_for(712) and len(e.slot_pages(1, a)) == 7      # never more than the ring
    assert e.free_pages(0) == 32 - 12 and e.free_pages(1) == 7
    e.slot_free(a)
    assert e.free_pages(0) == 32 and e.free_pages(1) == 14
    # a sequence no longer than a ring makes the group an ordinary one
    small = host_engine(max_tokens=64 * 8, max_seq_len=64 * 4, n_slots=2, layers=2, windows=(0, 100))
    assert small.kv_pages(1) == 8


def test_values_of_another_size_than_keys():
    from picolm_amd.parts import KVRequest
    assert KVRequest(2, 16, 0, 16) == KVRequest(2, 16) and KVRequest(2, 16).value_dim == 16
    assert KVRequest(2, 16, 0, 24) != KVRequest(2, 16) and KVRequest(2, 16, 0, 24).value_dim == 24
    e = host_engine(layers=1, v_head_dim=24)            # a called operation takes such a group; the attention operation does not
    a = e.slot_alloc()
    e.step([a], [[1] * 70])
    assert len(e.slot_pages(0, a)) == 2
    from picolm_amd.kernels import KernelError
    import torch
    from picolm_amd.cache import CacheSpec, KVGroupSpec
    from picolm_amd.engine import program as P
    from picolm_amd.engine.native import NativeEngine
    from picolm_amd.parts.base import CacheBinding
    b = P.ProgramBuilder(torch.float32, host_only=True)
    x = b.buffer("x", 96, torch.float32)
    b.embed(torch.zeros(10, 96), x)
    b.binding = CacheBinding((0, 0), None, True)
    b.attention(x, b.buffer("q", 64, torch.float32), b.buffer("o", 64, torch.float32), 4, 1, 16, 0, 0.25, None)
    lg = b.buffer("logits", 10, torch.float32, P.ROWS_WANTED)
    b.linear(torch.zeros(10, 96), b.buffer("h", 96, torch.float32, P.ROWS_WANTED), lg, 0, rows=P.ROWS_WANTED)
    b.logits_buffer = lg
    with pytest.raises(KernelError, match="keys and values of one size"):
        NativeEngine(b.finish(10, CacheSpec([KVGroupSpec(1, 1, 16, 0, 24)], [])), 64, 64, 1, "cpu", host_only=True)


def test_reservation_is_all_or_nothing_over_every_group():
    e = host_engine(max_tokens=64 * 8, max_seq_len=64 * 5, n_slots=4, layers=2, windows=(0, 100))
    a, b = e.slot_alloc(), e.slot_alloc()
    e.step([a], [[1] * 130])
    assert len(e.slot_pages(0, a)) == 3 and len(e.slot_pages(1, a)) == 3 and (e.length(a), e.length(b)) == (130, 0)
    with pytest.raises(CacheFull, match="exceeds"):
        e.step([b], [[1] * (64 * 5 + 1)])           # longer than a sequence may get
    with pytest.raises(CacheFull, match="more pages"):
        e.step([a, b], [[1] * 170, [1] * 300])      # 5 + 5 pages > 8
    assert len(e.slot_pages(0, a)) == 3 and e.slot_pages(0, b) == [] and e.slot_pages(1, b) == []
    e.step([a, b], [[1] * 70, [1] * 250])
    assert e.free_pages(0) == 0
    held = e.slot_pages(0, a) + e.slot_pages(0, b)
    assert sorted(held) == list(range(8))
    with pytest.raises(Exception, match="not live"):
        e.step([3], [[1] * 10])


def test_slots_are_given_back_and_used_again():
    e = host_engine(max_tokens=64 * 8, max_seq_len=64 * 5, n_slots=4, layers=2, windows=(0, 100), state_shape=(4, 2))
    a = e.slot_alloc()
    e.step([a], [[1] * 300])
    e.slot_free(a)
    assert e.free_pages(0) == 8 and e.free_pages(1) == 8
    with pytest.raises(CacheError, match="twice"):
        e.slot_free(a)
    assert e.free_pages(0) == 8                  # the refused free moved no page
    a2 = e.slot_alloc()
    assert a2 == a and e.length(a2) == 0
    assert e.state_bytes_per_slot(0) == 4 * 2 * 4


def test_random_walk_keeps_the_books_balanced():
    rnd = random.Random(0)
    e = host_engine(max_tokens=64 * 20, max_seq_len=64 * 8, n_slots=6, layers=2, windows=(0, 70))
    ring = min(window_ring_pages(70), 8)
    total = [e.kv_pages(0), e.kv_pages(1)]
    live = {}
    for _ in range(2000):
        op = rnd.random()
        if op < 0.3 and len(live) < 6:
            live[e.slot_alloc()] = 0
        elif op < 0.8 and live:
            s = rnd.choice(sorted(live))
            n = min(rnd.randint(1, 90), 64 * 8 - live[s])
            if n > 0:
                try:
                    e.step([s], [[1] * n])
                    live[s] += n
                except CacheFull:
                    pass
        elif live:
            s = rnd.choice(sorted(live))
            e.slot_free(s)
            del live[s]
        for g in (0, 1):
            held = [p for s in range(6) for p in e.slot_pages(g, s)]
            assert len(held) == len(set(held))                                  # no page held twice
            assert len(held) + e.free_pages(g) == total[g]                      # none lost
            for s in range(6):
                want = min(pages_for(live[s]), ring if g else 8) if s in live else 0
                assert len(e.slot_pages(g, s)) == want
        for s in range(6):
            assert e.length(s) == live.get(s, -1)
        assert e.info(2) + len(live) == 6
