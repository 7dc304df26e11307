"""The host side of a step: the packed description of a batch and the decode attention's
work list.  No GPU: the blocks are built on the CPU device."""
import numpy as np
import pytest

from picolm_amd.engine.batch import (DecodeBatch, StepBatch, StepError, decode_chunk_list,
                                     decode_pages_per_chunk)


def pages_of_list(pos0, window, ppc):
    """Every (sequence, page) the work list covers, by the arithmetic the kernels use."""
    seq, idx, most = decode_chunk_list(pos0, window, ppc)
    covered = []
    for s, i in zip(seq, idx):
        p = pos0[s]
        first = (max(0, p - window + 1) if window > 0 else 0) // 64
        end = p // 64 + 1
        lo = first + i * ppc
        hi = min(end, lo + ppc)
        assert lo < hi, "an empty chunk"
        assert i < most
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


def test_pages_per_chunk_grows_with_the_work():
    assert decode_pages_per_chunk([100], 8) == 4
    assert decode_pages_per_chunk([4095] * 8, 8) == 4
    big = decode_pages_per_chunk([4095] * 64, 8)
    assert big > 4 and big & (big - 1) == 0
    assert decode_pages_per_chunk([4095] * 64, 8, target_blocks=10 ** 9) == 4


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


def test_decode_batch_rewrites_its_lists_in_place():
    b = DecodeBatch(3, 4, "cpu")
    b.fill([2, 0, 1], [10, 300, 64], [1, 2, 3])
    seq, idx, cap, ppc, most = b.decode_chunks(8, 0, max_pages=16)
    assert cap == 3 * 4 and ppc == 4 and most == 4
    assert seq.tolist() == [0, 1, 1, 2] + [-1] * 8
    assert idx.tolist()[:4] == [0, 0, 1, 0]
    addr = seq.data_ptr()
    b.fill([2, 0, 1], [1000, 301, 65], [1, 2, 3])
    seq2, idx2, *_ = b.decode_chunks(8, 0, max_pages=16)
    assert seq2.data_ptr() == addr
    assert seq2.tolist() == [0, 0, 0, 0, 1, 1, 2] + [-1] * 5
    assert idx2.tolist()[:7] == [0, 1, 2, 3, 0, 1, 0]
    # a windowed layer has a list of its own
    wseq, *_ = b.decode_chunks(8, 64, max_pages=16)
    assert wseq.tolist()[:4] == [0, 1, 2, -1]
    with pytest.raises(StepError):
        b.fill([2, 0, 1], [1024, 0, 0], [1, 2, 3])       # 17 pages in a cache of 16
    b.frozen = True
    with pytest.raises(StepError):
        b.decode_chunks(8, 128, max_pages=16)
