"""The books and the step planning of the engine in the library (csrc/engine.hip), without a GPU:
an engine made with the host-only flag keeps slots, pages and page tables and plans every step's
index arrays, but holds no device memory and launches nothing.  Checked here: no slot or page is
lost, held twice or freed twice; a refused step changes nothing; the arrays of a step are those
of the plain planner (tests/plan_reference.py), which has tests of its own."""
import random

import numpy as np
import pytest
import torch

from host_engine import D, G, H, V, d, host_engine
from picolm_amd.cache import CacheError, CacheFull, CacheSpec
from picolm_amd.engine import StepError
from picolm_amd.engine import program as P
from picolm_amd.engine.native import NativeEngine
from plan_reference import StepBatch, decode_chunk_list, decode_pages_per_chunk, token_pages


def test_an_ill_formed_program_is_refused_with_the_operation_named():
    from picolm_amd.kernels import KernelError
    b = P.ProgramBuilder(torch.float32, host_only=True)
    x = b.buffer("residual", D, torch.float32)
    b.embed(torch.zeros(V, D), x)
    lg = b.buffer("logits", V, torch.float32, P.ROWS_WANTED)
    hf = b.buffer("norm.final", D + 8, torch.float32, P.ROWS_WANTED)
    b.linear(torch.zeros(V, D + 16), hf, lg, 0, rows=P.ROWS_WANTED)         # reads rows wider than its input buffer
    b.logits_buffer = lg
    with pytest.raises(KernelError, match="operation 1 .product. reads rows of 80 values"):
        NativeEngine(b.finish(V, CacheSpec([], [])), 64, 64, 1, "cpu", host_only=True)
    with pytest.raises(CacheError, match="positive"):
        host_engine(max_tokens=0)
    # a norm is prepared for every row of the step or not at all
    b = P.ProgramBuilder(torch.float32, host_only=True)
    x = b.buffer("residual", D, torch.float32)
    b.embed(torch.zeros(V, D), x)
    few = b.buffer("few", D, torch.float32, P.ROWS_WANTED)
    acc = b.buffer("acc", D, torch.float32, P.ROWS_WANTED)
    b.linear(torch.zeros(D, D), few, acc, 1, rows=P.ROWS_WANTED, out_norm=P.NormRef(torch.ones(D), 1e-5))
    lg = b.buffer("logits", V, torch.float32, P.ROWS_WANTED)
    b.linear(torch.zeros(V, D), acc, lg, 0, rows=P.ROWS_WANTED)
    b.logits_buffer = lg
    with pytest.raises(KernelError, match="operation 1: only a product over every row of the step prepares a norm"):
        NativeEngine(b.finish(V, CacheSpec([], [])), 64, 64, 1, "cpu", host_only=True)


def test_a_called_operation_on_a_ring_is_given_no_more_than_the_ring_takes_in():
    """The attention operation answers a long prompt over a window slice by slice; a called
    operation sees a step whole, so a step that its ring cannot take in at once is refused
    before anything moves."""
    e = host_engine(max_tokens=64 * 40, max_seq_len=1024, n_slots=2, layers=2, windows=(0, 100), v_head_dim=16)
    a, b = e.slot_alloc(), e.slot_alloc()
    free = [e.free_pages(0), e.free_pages(1)]
    with pytest.raises(StepError, match="up to 256 tokens a sequence, sequence 1 brings 257"):
        e.step([a, b], [[1] * 10, [2] * 257])
    assert [e.free_pages(0), e.free_pages(1)] == free and (e.length(a), e.length(b)) == (0, 0)
    e.step([a, b], [[1] * 10, [2] * 256])
    e.step([a, b], [[1] * 256, [2] * 200])                  # and goes on in further steps
    assert (e.length(a), e.length(b)) == (266, 456)
    whole = host_engine(max_tokens=64 * 40, max_seq_len=1024, n_slots=2, layers=2, windows=(0,), v_head_dim=16)
    s = whole.slot_alloc()
    whole.step([s], [[1] * 700])                             # no ring: any length


def test_slots_and_pages_are_handed_out_and_taken_back():
    e = host_engine()
    assert [e.info(i) for i in (0, 1, 2, 3, 5)] == [256, 3, 3, 640, 4]      # max_seq_len, slots, free slots, free tokens, pages a row
    # keys and values: two entries of ten pages of G x 64 x d floats, twice; no state here, and one with state
    assert e.info(9) == 2 * 2 * 10 * G * 64 * d * 4 and e.info(8) == 0
    assert host_engine(state_shape=(4, 2)).info(9) == e.info(9) + 2 * 3 * 8 * 4
    a, b, c = e.slot_alloc(), e.slot_alloc(), e.slot_alloc()
    assert (a, b, c) == (0, 1, 2)
    with pytest.raises(CacheFull, match="all 3 slots"):
        e.slot_alloc()
    e.step([a, b], [[1] * 70, [2] * 5])
    assert e.slot_pages(0, a) == [0, 1] and e.slot_pages(0, b) == [2] and e.free_pages(0) == 7
    assert (e.length(a), e.length(b), e.length(c)) == (70, 5, 0)
    e.slot_free(b)
    assert e.free_pages(0) == 8 and e.length(b) == -1
    with pytest.raises(CacheError, match="freed twice"):
        e.slot_free(b)
    with pytest.raises(CacheError, match="does not exist"):
        e.slot_free(7)
    assert e.free_pages(0) == 8                       # the refused calls moved nothing
    assert e.slot_alloc() == b and e.length(b) == 0   # used again, from nothing
    e.step([b], [[3] * 64])
    assert e.slot_pages(0, b) == [2]                  # the page that was given back, first


def test_a_refused_step_leaves_everything_where_it_was():
    e = host_engine()
    a, b = e.slot_alloc(), e.slot_alloc()
    e.step([a, b], [[1] * 100, [2] * 100])
    before = (e.free_pages(0), e.slot_pages(0, a), e.slot_pages(0, b), e.length(a), e.length(b), e.info(7))
    with pytest.raises(CacheFull, match="exceeds"):
        e.step([a, b], [[1] * 10, [2] * 157])         # the second would hold 257 of 256
    with pytest.raises(StepError, match="vocabulary"):
        e.step([a], [[1, V]])
    with pytest.raises(StepError, match="twice"):
        e.step([a, a], [[1], [2]])
    with pytest.raises(StepError, match="not live"):
        e.step([2], [[1]])
    with pytest.raises(StepError, match="wanted row 3"):
        e.step([a], [[1, 2, 3]], [[3]])
    assert before == (e.free_pages(0), e.slot_pages(0, a), e.slot_pages(0, b), e.length(a), e.length(b), e.info(7))
    full = host_engine(max_tokens=64 * 3, n_slots=3)
    x, y = full.slot_alloc(), full.slot_alloc()
    full.step([x], [[1] * 128])
    with pytest.raises(CacheFull, match="more pages"):
        full.step([x, y], [[1], [2] * 65])            # one page for x's 129th token, two for y: three, and one is free
    assert full.free_pages(0) == 1 and full.length(x) == 128 and full.slot_pages(0, y) == []


def test_random_walk_keeps_the_books_balanced():
    rnd = random.Random(1)
    e = host_engine(max_tokens=64 * 20, max_seq_len=64 * 8, n_slots=6, layers=1)
    live = {}
    for _ in range(1500):
        op = rnd.random()
        if op < 0.25 and len(live) < 6:
            live[e.slot_alloc()] = 0
        elif op < 0.8 and live:
            who = rnd.sample(sorted(live), rnd.randint(1, len(live)))
            if rnd.random() < 0.5:
                news = [1] * len(who)
            else:
                news = [rnd.randint(1, 90) for _ in who]
            try:
                e.step(who, [[1] * n for n in news])
                for s, n in zip(who, news):
                    live[s] += n
            except CacheFull:
                pass
        elif live:
            s = rnd.choice(sorted(live))
            e.slot_free(s)
            del live[s]
        held = [p for s in range(6) for p in e.slot_pages(0, s)]
        assert len(held) == len(set(held))                                   # no page held twice
        assert len(held) + e.free_pages(0) == 20                             # none lost
        for s in range(6):
            assert len(e.slot_pages(0, s)) == ((live[s] + 63) // 64 if s in live else 0)
            assert e.length(s) == live.get(s, -1)
        assert e.info(2) + len(live) == 6


def table_of(e, n_slots, max_pages, group=0):
    t = np.zeros((n_slots, max_pages), dtype=np.int32)
    for s in range(n_slots):
        pages = e.slot_pages(group, s)
        t[s, :len(pages)] = pages
    return t


def test_a_prefill_step_is_planned_as_the_plain_planner_plans_it():
    e = host_engine(max_tokens=64 * 40, max_seq_len=64 * 8, n_slots=4)
    slots = [e.slot_alloc() for _ in range(4)]
    order = [slots[2], slots[0], slots[3]]
    e.step([slots[1]], [[5] * 30])                    # so that pages are not simply in the slots' order
    first = [[1] * 70, [2] * 5, [3] * 130]
    e.step(order, first, [[0, 69], [], [129]])
    more = [[4] * 40, [5], [6] * 100]                 # onto what the slots hold
    want = [[39], [0], [0, 99]]
    e.step(order, more, want)
    pos0 = [70, 5, 130]
    ref = StepBatch(order, pos0, more, want, V, "cpu")
    for name in ("seq_slot", "seq_pos0", "seq_nnew", "cu_seqlens", "tok_pos", "tok_seq", "tokens", "want_rows"):
        assert np.array_equal(e.step_array(name), getattr(ref, name).numpy()[:len(e.step_array(name))]), name
    table = table_of(e, 4, 8)
    assert np.array_equal(e.step_array("write_pages.0"), token_pages(ref._host["tok_seq"], ref._host["tok_pos"], order, table, 8))
    seq, q0, n = ref.prefill_tiles(16)
    assert np.array_equal(e.step_array("tiles.16.seq"), seq.numpy()) and np.array_equal(e.step_array("tiles.16.q0"), q0.numpy())
    assert [e.length(s) for s in order] == [110, 6, 230]


@pytest.mark.parametrize("lengths", [[70, 5, 130], [500, 1, 64, 63], [507] * 4, [300] * 40])
def test_a_decode_step_is_planned_as_the_plain_planner_plans_it(lengths):
    n = len(lengths)
    e = host_engine(max_tokens=64 * 8 * n, max_seq_len=512, n_slots=n)
    slots = [e.slot_alloc() for _ in range(n)]
    e.step(slots, [[1] * L for L in lengths])
    for step in range(3):                             # the first builds the lists, the others move on in place
        pos0 = [L + step for L in lengths]
        e.step(slots, [[7 + i] for i in range(n)])
        table = table_of(e, n, 8)
        ppc = decode_pages_per_chunk(pos0, G * 1, 16)            # one workgroup per KV head and chunk in the float kernels
        entries, most = decode_chunk_list(slots, pos0, 0, ppc, table, 8)
        got = e.step_array("chunks.0").reshape(-1, 8)
        assert got[0, 0] == len(entries)
        assert np.array_equal(got[1:1 + len(entries)], entries)
        assert np.array_equal(e.step_array("tok_pos"), pos0) and np.array_equal(e.step_array("seq_slot"), slots)
        assert np.array_equal(e.step_array("tokens"), [7 + i for i in range(n)])
        assert np.array_equal(e.step_array("write_pages.0"), token_pages(np.arange(n), pos0, slots, table, 8))
    # a decode step that does not want every row is planned like any other step, with the same list
    pos0 = [L + 3 for L in lengths]
    e.step(slots, [[1]] * n, [[0]] * (n - 1) + [[]])
    entries, _ = decode_chunk_list(slots, pos0, 0, decode_pages_per_chunk(pos0, G, 16), table_of(e, n, 8), 8)
    got = e.step_array("chunks.0").reshape(-1, 8)
    assert got[0, 0] == len(entries) and np.array_equal(got[1:], entries)
    assert np.array_equal(e.step_array("want_rows"), np.arange(n - 1))


def test_a_slot_that_changes_hands_is_looked_up_again_by_the_decode_step():
    e = host_engine(max_tokens=64 * 12, max_seq_len=256, n_slots=3)
    a, b = e.slot_alloc(), e.slot_alloc()
    e.step([a, b], [[1] * 10, [2] * 20])
    e.step([a, b], [[1], [2]])
    first = e.step_array("chunks.0").reshape(-1, 8).copy()
    e.slot_free(a)
    c = e.slot_alloc()                                 # holds what `a` held, in another slot's place
    hold = e.slot_alloc()
    e.step([hold], [[3] * 70])                         # takes the page that `a` gave back
    assert c == a
    e.step([c], [[4] * 11])                            # as long as `a` was one step ago, on other pages
    e.step([c, b], [[1], [2]])                         # looks like the next step of the old pair
    second = e.step_array("chunks.0").reshape(-1, 8)
    assert second[0, 0] == 2
    rows = {int(r[0]): r for r in second[1:3]}
    assert rows[0][2] == 11 and rows[0][4] == e.slot_pages(0, c)[0] != first[1 + list(first[1:3, 0]).index(0)][4]
    assert np.array_equal(e.step_array("write_pages.0"), [e.slot_pages(0, c)[0], e.slot_pages(0, b)[0]])


@pytest.mark.parametrize("window", [1, 64, 100, 200])
def test_a_decode_step_over_a_window_is_planned_as_the_plain_planner_plans_it(window):
    """A group that keeps a window of keys: the work list covers the pages of the last `window` keys
    only, its first page moves with every step, and pages lie in the slot's ring.  Walked over 150
    steps (page boundaries, laps of the ring), in the block that stays in place."""
    from picolm_amd.cache import window_ring_pages
    lengths = [500, 3, 130]
    e = host_engine(max_tokens=64 * 64, max_seq_len=1024, n_slots=3, layers=2, windows=(0, window))
    ring = min(window_ring_pages(window), 16)
    slots = [e.slot_alloc() for _ in range(3)]
    for lo in range(0, 500, 250):
        live = [i for i in range(3) if lengths[i] > lo]
        e.step([slots[i] for i in live], [[1] * min(250, lengths[i] - lo) for i in live])
    for step in range(150):
        pos0 = [L + step for L in lengths]
        e.step(slots, [[7]] * 3)
        ppc = decode_pages_per_chunk(pos0, G, 16)
        for group, (w, r) in enumerate(((0, 16), (window, ring))):
            entries, _ = decode_chunk_list(slots, pos0, w, ppc, table_of(e, 3, 16, group), r)
            got = e.step_array(f"chunks.{group}").reshape(-1, 8)
            assert got[0, 0] == len(entries) and np.array_equal(got[1:1 + len(entries)], entries), (step, group)
            assert np.array_equal(e.step_array(f"write_pages.{group}"), token_pages(np.arange(3), pos0, slots, table_of(e, 3, 16, group), r))
        assert all(len(e.slot_pages(1, s)) <= ring for s in slots)


def test_a_long_prefill_step_over_a_window_is_cut_along_positions():
    """Where a group keeps a ring, a step of more than 256 tokens a sequence is planned a second
    time as slices of 256 positions, each with sequences, rows and tiles of its own."""
    e = host_engine(max_tokens=64 * 64, max_seq_len=1024, n_slots=3, layers=2, windows=(0, 100))
    slots = [e.slot_alloc() for _ in range(3)]
    e.step([slots[1]], [[1] * 40])
    news = [[1] * 700, [2] * 30, [3] * 257]
    e.step(slots, news)
    ref = StepBatch(slots, [0, 40, 0], news, [[], [], []], V, "cpu")
    chunks = list(ref.chunks(256))
    assert len(chunks) == 3
    for c, want in enumerate(chunks):
        for name, have in (("seq_slot", want.seq_slot), ("seq_pos0", want.seq_pos0), ("seq_nnew", want.seq_nnew),
                           ("first_row", want.cu_seqlens), ("rows", want.rows)):
            assert np.array_equal(e.step_array(f"window_chunk.{c}.{name}"), have.numpy()[:len(e.step_array(f"window_chunk.{c}.{name}"))]), (c, name)
        seq, q0, n = want.prefill_tiles(16)
        assert np.array_equal(e.step_array(f"window_chunk.{c}.tiles.16.seq"), seq.numpy())
        assert np.array_equal(e.step_array(f"window_chunk.{c}.tiles.16.q0"), q0.numpy())
    with pytest.raises(Exception, match="no array"):
        e.step_array("window_chunk.3.rows")
    e.step(slots, [[1] * 200, [2] * 256, [3] * 9])          # no sequence brings more than 256: no slices
    with pytest.raises(Exception, match="no array"):
        e.step_array("window_chunk.0.rows")


def test_more_shapes_of_decode_steps_than_the_engine_keeps():
    """The engine keeps the blocks (and recordings) of 48 shapes of decode steps and lets the least
    recently used go: batches of 1 to 60 sequences in turn, then the first shapes again, are all
    planned as the plain planner plans them."""
    n_slots = 60
    e = host_engine(max_tokens=64 * 4 * n_slots, max_seq_len=256, n_slots=n_slots)
    slots = [e.slot_alloc() for _ in range(n_slots)]
    e.step(slots, [[1] * (3 + i % 5) for i in range(n_slots)])
    length = [3 + i % 5 for i in range(n_slots)]
    for n in list(range(1, n_slots + 1)) + [1, 2, 3, 60, 30]:
        for _ in range(2):
            pos0 = length[:n]
            e.step(slots[:n], [[9 + i] for i in range(n)])
            table = table_of(e, n_slots, 4)
            ppc = decode_pages_per_chunk(pos0, G, 16)
            entries, _ = decode_chunk_list(slots[:n], pos0, 0, ppc, table, 4)
            got = e.step_array("chunks.0").reshape(-1, 8)
            assert got[0, 0] == len(entries) and np.array_equal(got[1:1 + len(entries)], entries), n
            assert np.array_equal(e.step_array("tok_pos"), pos0) and np.array_equal(e.step_array("seq_slot"), slots[:n])
            assert np.array_equal(e.step_array("write_pages.0"), token_pages(np.arange(n), pos0, slots[:n], table, 4))
            for i in range(n):
                length[i] += 1
    assert [e.length(s) for s in slots] == length
