"""The plain planner of a step's index arrays (tests/plan_reference.py), pinned by cases worked out
by hand: the packed description of a batch, the decode attention's work list, every token's cache
page, the prefill's tiles.  The engine's own planning is held to it in test_engine_books.py."""
import numpy as np
import pytest

from plan_reference import StepBatch, StepError, decode_chunk_list, decode_pages_per_chunk


def make_table(pos0, ring_pages, seed=0):
    """A page table with distinct physical pages for every (slot, ring position)."""
    rng = np.random.default_rng(seed)
    slots = list(rng.permutation(len(pos0) + 3)[:len(pos0)])
    table = rng.permutation((len(pos0) + 3) * ring_pages).astype(np.int32).reshape(len(pos0) + 3, ring_pages)
    return slots, table


def pages_of_list(pos0, window, ppc, ring_pages=64):
    """Every (sequence, page) the work list covers, by the arithmetic the kernels use."""
    slots, table = make_table(pos0, ring_pages)
    entries, most = decode_chunk_list(slots, pos0, window, ppc, table, ring_pages)
    covered = []
    for s, i, qpos, slot, *phys in entries:
        assert qpos == pos0[s] and slot == slots[s]
        first = (max(0, qpos - window + 1) if window > 0 else 0) // 64
        end = qpos // 64 + 1
        lo = first + i * ppc
        hi = min(end, lo + ppc)
        assert lo < hi, "an empty chunk"
        assert i < most
        for w in range(4):
            want = table[slot, (lo + w) % ring_pages] if lo + w < hi else -1
            assert phys[w] == want
        covered += [(int(s), page) for page in range(lo, hi)]
    return covered


@pytest.mark.parametrize("window", [0, 1, 64, 100, 1000])
@pytest.mark.parametrize("ppc", [1, 3, 4, 64])
def test_work_list_covers_every_visible_page_once(window, ppc):
    pos0 = [0, 63, 64, 127, 128, 700, 4095, 129]
    covered = pages_of_list(pos0, window, ppc)
    expect = []
    for s, p in enumerate(pos0):
        lo = max(0, p - window + 1) if window > 0 else 0
        expect += [(s, page) for page in range(lo // 64, p // 64 + 1)]
    assert sorted(covered) == sorted(expect)
    assert len(set(covered)) == len(covered)


def test_work_list_of_a_ring():
    """A windowed group keeps a ring of pages: page p lives at ring position p % ring_pages."""
    covered = pages_of_list([5000, 100], 200, 2, ring_pages=9)
    assert sorted(covered) == [(0, p) for p in range(75, 79)] + [(1, 0), (1, 1)]


def test_pages_per_chunk_grows_with_the_work():
    assert decode_pages_per_chunk([100], 8) == 4                       # too little work for larger chunks
    assert decode_pages_per_chunk([1100] * 8, 8) == 8                  # 18 pages each: 3 chunks of 8 x 8 x 8 = 192 workgroups
    assert decode_pages_per_chunk([4095] * 8, 8) == 16
    assert decode_pages_per_chunk([4095] * 8, 8, max_pages_per_chunk=8) == 8
    assert decode_pages_per_chunk([1100] * 64, 8, max_pages_per_chunk=8) == 8
    assert decode_pages_per_chunk([4095] * 64, 8, min_blocks=10 ** 9) == 4


def test_step_batch_packs_without_padding():
    b = StepBatch([3, 1], [0, 0], [[5, 6, 7], [8]], [[0, 2], []], 10, "cpu")
    assert b.T == 4 and not b.is_decode and b.n_want == 2
    assert b.cu_seqlens.tolist() == [0, 3, 4]
    assert b.tok_pos.tolist()[:4] == [0, 1, 2, 0]
    assert b.tok_seq.tolist()[:4] == [0, 0, 0, 1]
    assert b.want_rows.tolist()[:2] == [0, 2]
    with pytest.raises(StepError):
        StepBatch([1, 1], [0, 0], [[1], [2]], [[0], [0]], 10, "cpu")
    with pytest.raises(StepError):
        StepBatch([1], [0], [[10]], [[0]], 10, "cpu")
    with pytest.raises(StepError):
        StepBatch([1], [0], [[1]], [[1]], 10, "cpu")


def test_write_pages_follow_the_page_table():
    table = np.arange(3 * 5, dtype=np.int32).reshape(3, 5) + 100
    b = StepBatch([2, 0], [61, 0], [[1] * 5, [2] * 70], [[], []], 10, "cpu")
    pages = b.write_pages(0, table, 5).tolist()
    assert pages[:5] == [110, 110, 110, 111, 111]            # slot 2: positions 61..65
    assert pages[5:5 + 64] == [100] * 64 and pages[69:75] == [101] * 6
    ring = b.write_pages(1, table, 1).tolist()                 # a ring of one page
    assert ring[:5] == [110] * 5 and ring[5:] == [100] * 70


def test_prefill_tiles_are_listed_by_the_keys_they_see():
    """Fewest keys first (the kernels hand out the longest first); every tile once."""
    b = StepBatch([0, 1, 2], [100, 0, 5], [[1] * 70, [1] * 200, [1] * 33], [[], [], []], 10, "cpu")
    seq, q0, n = b.prefill_tiles(32)
    tiles = list(zip(seq.tolist(), q0.tolist()))
    assert n == 3 + 7 + 2 and sorted(tiles) == sorted((i, q) for i, m in enumerate([70, 200, 33]) for q in range(0, m, 32))
    ends = [[100, 0, 5][i] + min(q + 32, [70, 200, 33][i]) for i, q in tiles]
    assert ends == sorted(ends)
    for c in b.chunks(64):                       # a step cut along positions lists its own tiles
        seq_c, q0_c, n_c = c.prefill_tiles(32)
        assert n_c == sum((m + 31) // 32 for m in c.n_new)
