"""The host side of a step: the packed description of a batch and the decode attention's
work list.  No GPU: the blocks are built on the CPU device."""
import numpy as np
import pytest

from picolm_amd.engine.batch import (DecodeBatch, StepBatch, StepError, decode_chunk_list,
                                     decode_pages_per_chunk)


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


def test_decode_batch_rewrites_its_lists_in_place():
    import torch
    table = torch.arange(4 * 16, dtype=torch.int32).reshape(4, 16)
    b = DecodeBatch(3, 4, "cpu")
    b.fill([2, 0, 1], [10, 300, 64], [1, 2, 3])
    dev, cap, ppc, most = b.decode_chunks(8, 16, 0, 0, table, 16)
    assert cap == 3 * 4 and ppc == 4 and most == 4
    assert dev.reshape(-1, 8)[0, 0] == 4                    # the header: entries in use
    # the chunks with the most pages come first; every entry says whose it is
    assert dev.reshape(-1, 8)[1:5, :2].tolist() == [[1, 0], [2, 0], [0, 0], [1, 1]]
    rows = torch.tensor(sorted(dev.reshape(-1, 8)[1:5].tolist()))          # by sequence and chunk
    assert rows[:4, 0].tolist() == [0, 1, 1, 2]
    assert rows[:4, 1].tolist() == [0, 0, 1, 0]
    assert rows[:4, 2].tolist() == [10, 300, 300, 64]
    assert rows[:4, 3].tolist() == [2, 0, 0, 1]
    assert rows[1, 4:].tolist() == [0, 1, 2, 3] and rows[2, 4:].tolist() == [4, -1, -1, -1]
    assert rows[0, 4:].tolist() == [32, -1, -1, -1]
    addr = dev.data_ptr()
    b.fill([2, 0, 1], [1000, 301, 65], [1, 2, 3])
    dev2, *_ = b.decode_chunks(8, 16, 0, 0, table, 16)
    assert dev2.data_ptr() == addr
    assert dev2.reshape(-1, 8)[0, 0] == 7
    rows = torch.tensor(sorted(dev2.reshape(-1, 8)[1:8].tolist()))
    assert rows[:7, 0].tolist() == [0, 0, 0, 0, 1, 1, 2]
    assert rows[:7, 1].tolist() == [0, 1, 2, 3, 0, 1, 0]
    # a windowed layer, or another cache group, has a list of its own
    wdev, *_ = b.decode_chunks(8, 16, 64, 0, table, 16)
    assert wdev.reshape(-1, 8)[0, 0] == 3 and sorted(wdev.reshape(-1, 8)[1:4, 0].tolist()) == [0, 1, 2]
    pages = b.write_pages(0, table, 16)
    assert pages.tolist() == [32 + 15, 4, 16 + 1]          # positions 1000, 301, 65 of slots 2, 0, 1
    b.fill([2, 0, 1], [64, 0, 128], [1, 2, 3])
    assert pages.tolist() == [33, 0, 18]
    with pytest.raises(StepError):
        b.fill([2, 0, 1], [1024, 0, 0], [1, 2, 3])       # 17 pages in a cache of 16
    b.frozen = True
    with pytest.raises(StepError):
        b.decode_chunks(8, 16, 128, 0, table, 16)


def test_decode_batch_between_page_boundaries_only_moves_positions():
    """Filling step by step (the short way when no sequence starts a page) gives the same blocks
    as filling a fresh batch; a step that starts a page rebuilds the lists."""
    import torch
    table = torch.from_numpy(np.random.default_rng(0).permutation(4 * 16).astype(np.int32).reshape(4, 16))
    slots = [2, 0, 1]
    walked = DecodeBatch(3, 4, "cpu", reserve_ints=2 * DecodeBatch.ints_for(3, 4, 16))
    pos = [60, 300, 125]
    walked.fill(slots, pos, [1, 2, 3], cache_version=7)
    lists = [walked.decode_chunks(8, 16, w, 0, table, 16)[0] for w in (0, 100)]
    pages = walked.write_pages(0, table, 16)
    for step in range(1, 8):                     # positions 64 and 128 start pages on the way
        pos = [p + 1 for p in pos]
        walked.fill(slots, pos, [step] * 3, cache_version=7)
        fresh = DecodeBatch(3, 4, "cpu")
        fresh.fill(slots, pos, [step] * 3)
        for w, got in zip((0, 100), lists):
            want = fresh.decode_chunks(8, 16, w, 0, table, 16)[0]
            n = int(want.reshape(-1, 8)[0, 0])
            assert got.reshape(-1, 8)[:n + 1].tolist() == want.reshape(-1, 8)[:n + 1].tolist(), (step, w)
        assert pages.tolist() == fresh.write_pages(0, table, 16).tolist()
        assert walked.seq_pos0.tolist() == pos and walked.tokens.tolist() == [step] * 3


def test_decode_batch_looks_pages_up_again_when_the_cache_changed():
    """The same slots one position further, but the slots changed hands in between (another batch
    got them): the page ids of the last fill are stale and must not be kept."""
    import torch
    table = torch.arange(2 * 8, dtype=torch.int32).reshape(2, 8).clone()
    b = DecodeBatch(2, 4, "cpu", reserve_ints=DecodeBatch.ints_for(2, 4, 8))
    b.fill([0, 1], [10, 70], [1, 1], cache_version=3)
    dev = b.decode_chunks(8, 16, 0, 0, table, 8)[0]
    pages = b.write_pages(0, table, 8)
    table += 100                                        # other pages now
    b.fill([0, 1], [11, 71], [1, 1], cache_version=4)
    assert pages.tolist() == [100, 109]
    assert sorted(dev.reshape(-1, 8)[1:3].tolist())[0][4] == 100          # sequence 0's first page
    b.fill([0, 1], [12, 72], [1, 1], cache_version=4)   # nothing changed: positions only
    assert sorted(dev.reshape(-1, 8)[1:3, 2].tolist()) == [12, 72] and pages.tolist() == [100, 109]
    table += 100
    b.fill([0, 1], [13, 73], [1, 1])                    # no version given: never the short way
    assert pages.tolist() == [200, 209]


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
