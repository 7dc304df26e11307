"""The engine behind the C ABI (csrc/engine.h).  Its entry points are called through ctypes as a C
program would call them, over the three ways of cutting the work (each request whole; its last
tokens one by one; unequal batches one after another in slots that are used again), against the
plain implementation; its generation loop makes the tokens that the Python loop makes, and the
tokens that the plain sampler draws from the plain logits."""
import ctypes
from ctypes import byref, c_int32, c_void_p

import numpy as np
import pytest
import torch

import tiny

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


tolerance = tiny.tolerance


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("models")
    return {w: tiny.make_model_dir(tmp, w) for w in tiny.CONFIGS}


class CEngine:
    """picolm_engine_* through ctypes, nothing else: arrays go in as pointers, logits come back as a
    device pointer that is copied to the host with hipMemcpy."""

    def __init__(self, model, max_tokens, n_slots=0, flags=0):
        from picolm_amd import kernels
        from picolm_amd.engine import program as P
        self.lib = kernels.lib()
        P.declare(self.lib)
        model.prepare(model.config.max_position_embeddings)
        self.built = model.program()
        self.V = model.head.V
        self.h = c_void_p()
        rc = self.lib.picolm_engine_create(byref(self.built.struct), max_tokens, model.config.max_position_embeddings, n_slots,
                                           flags, byref(self.h))
        assert rc == 0, self.lib.picolm_last_error()
        self.hip = ctypes.CDLL("libamdhip64.so")

    def alloc(self):
        s = c_int32(-1)
        rc = self.lib.picolm_engine_slot_alloc(self.h, byref(s), None)
        assert rc == 0, self.lib.picolm_last_error()
        return s.value

    def free(self, slot):
        return self.lib.picolm_engine_slot_free(self.h, slot)

    def step(self, slots, tokens, want=None):
        arr = lambda v: np.ascontiguousarray(v, dtype=np.int32)
        sl, nn, flat = arr(slots), arr([len(t) for t in tokens]), arr([x for t in tokens for x in t])
        counts = idx = None
        if want is not None:
            counts, idx = arr([len(w) for w in want]), arr([j for w in want for j in w] or [0])
        logits, rows = c_void_p(), c_int32()
        rc = self.lib.picolm_engine_step(self.h, len(sl), sl.ctypes.data, nn.ctypes.data, flat.ctypes.data,
                                         counts.ctypes.data if want is not None else None,
                                         idx.ctypes.data if want is not None else None, byref(logits), byref(rows), None)
        if rc:
            return rc
        out = np.empty((rows.value, self.V), dtype=np.float32)
        if rows.value:
            assert self.hip.hipMemcpy(c_void_p(out.ctypes.data), logits, ctypes.c_size_t(out.nbytes), 2) == 0    # device to host
        return out

    def close(self):
        self.lib.picolm_engine_destroy(self.h)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "D", "F"])
def test_the_c_entry_points_over_the_three_cuttings(which, dtype, folders):
    from picolm_amd.engine import load_model
    d = folders[which]
    V = tiny.read_config(d)["vocab_size"]
    rng = np.random.default_rng(40)
    reqs = [tiny.random_tokens(rng, n, V) for n in (33, 47, 64, 65, 100, 128)]
    truth = [tiny.plain_logits(d, r) for r in reqs]
    room = sum((len(r) + 63) // 64 for r in reqs[3:]) * 64              # the larger batch only
    e = CEngine(load_model(d, dtype=dtype), room, n_slots=3)

    def check(got, ref, what):
        assert not isinstance(got, int), (what, e.lib.picolm_last_error())
        err = float(np.abs(got.astype(np.float64) - ref).max())
        assert err <= tolerance(dtype, ref), f"{which} {dtype} {what}: {err}"
    for i, r in enumerate(reqs):                                        # whole
        s = e.alloc()
        check(e.step([s], [r], [list(range(len(r)))]), truth[i], f"whole {i}")
        assert e.free(s) == 0
    for i, r in enumerate(reqs):                                        # the last 32 tokens one by one
        s, n0 = e.alloc(), len(r) - 32
        check(e.step([s], [r[:n0]]), truth[i][n0 - 1:n0], f"tail {i} prompt")
        for j in range(n0, len(r)):
            check(e.step([s], [[r[j]]]), truth[i][j:j + 1], f"tail {i} position {j}")
        assert e.free(s) == 0
    for ids in ([0, 1, 2], [3, 4, 5]):                                  # unequal batches, slots used again
        n_dec = dict(zip(ids, (3, 9, 20)))
        pos = {i: len(reqs[i]) - n_dec[i] for i in ids}
        slot = {i: e.alloc() for i in ids}
        assert sorted(slot.values()) == [0, 1, 2]
        got = e.step([slot[i] for i in ids], [reqs[i][:pos[i]] for i in ids], [[0, pos[i] - 1] for i in ids])
        for k, i in enumerate(ids):
            check(got[2 * k:2 * k + 2], truth[i][[0, pos[i] - 1]], f"batch prompt {i}")
        live = list(ids)
        while live:
            got = e.step([slot[i] for i in live], [[reqs[i][pos[i]]] for i in live])
            for k, i in enumerate(live):
                check(got[k:k + 1], truth[i][pos[i]:pos[i] + 1], f"batch decode {i} at {pos[i]}")
                pos[i] += 1
            for i in [i for i in live if pos[i] == len(reqs[i])]:
                assert e.free(slot[i]) == 0
                live.remove(i)
    # refusals come back as codes with a message, and leave the sequence where it was
    s = e.alloc()
    assert e.step([s], [[V]]) == -10 and b"vocabulary" in e.lib.picolm_last_error()
    assert e.step([s, s], [[1], [2]]) == -10 and b"twice" in e.lib.picolm_last_error()
    assert e.step([s], [[1] * 4000]) == -11
    assert e.lib.picolm_engine_slot_length(e.h, s) == 0
    assert e.free(s) == 0 and e.free(s) == -12 and b"twice" in e.lib.picolm_last_error()
    e.close()


@pytest.mark.parametrize("params", [(0.0, 0, 1.0, 0.0, 42), (0.8, 40, 0.9, 0.05, 7), (1.1, 0, 1.0, 0.0, 0)])
def test_the_library_loop_makes_the_tokens_of_the_python_loop(params, folders):
    from picolm_amd import SamplingParams, generate
    from picolm_amd.engine import Session, load_model
    d = folders["B"]
    V = tiny.TINY_B["vocab_size"]
    model = load_model(d, dtype="bfloat16")
    rng = np.random.default_rng(42)
    prompts = [tiny.random_tokens(rng, n, V) for n in (1, 9, 30, 64, 17, 3, 100)]
    sp = SamplingParams(*params)
    free = generate(Session(model, max_tokens=4 * 192), prompts, 25, sp, stop_ids=[], batch_size=3)
    stop = [free[0].tokens[10], free[4].tokens[3]]         # tokens that do come: some sequences stop early, others do not
    want = generate(Session(model, max_tokens=4 * 192), prompts, 25, sp, stop_ids=stop, batch_size=3)
    s = Session(model, max_tokens=4 * 192)
    toks, finish = s.engine.generate(prompts, 25, sp, stop, batch_size=3)
    assert toks == [r.tokens for r in want]
    assert finish == [r.finish for r in want]
    assert any(f == "stop" for f in finish) and any(f == "length" for f in finish)
    assert s.cache.slots.n_free == s.cache.n_slots
    # a sequence that reaches the cache's capacity ends there
    small = Session(model, max_tokens=128, max_seq_len=70)
    toks, finish = small.engine.generate([prompts[3]], 25, SamplingParams(), [], batch_size=1)
    assert finish == ["capacity"] and len(toks[0]) == 70 - 64 + 1


@pytest.mark.parametrize("params", [(0.0, 0, 1.0, 0.0, 42), (0.8, 40, 0.9, 0.05, 7)])
def test_the_library_loop_against_the_plain_sampler_at_matrix_core_sizes(params, folders):
    """picolm_engine_generate on configuration E (width 1,024, heads of 128, four query heads a KV
    head: the sizes the matrix-core kernels are made for), batches of three after one another with
    stop tokens.  In 32-bit every token is what the plain sampler draws from the plain logits of
    the sequence so far, with that request's generator stream.  In bfloat16 (greedy) every token's
    plain logit lies within the engine's distance of the largest."""
    from plain import sampler_plain as SP
    from picolm_amd import SamplingParams
    from picolm_amd.engine import Session, load_model
    from picolm_amd.sampling import stream_state
    from plain import llama_plain
    d = folders["E"]
    V = tiny.TINY_E["vocab_size"]
    weights, config = tiny.read_weights_f64(d), tiny.read_config(d)
    plain_logits = lambda seq: llama_plain.forward(weights, config, seq)
    rng = np.random.default_rng(44)
    prompts = [tiny.random_tokens(rng, n, V) for n in (1, 70, 9, 130, 33, 64, 65)]
    sp = SamplingParams(*params)
    n_new = 10
    model = load_model(d, dtype="float32")
    free, _ = Session(model, max_tokens=3 * 256).engine.generate(prompts, n_new, sp, [], batch_size=3)
    stop = [free[1][4], free[5][7]]
    toks, finish = Session(model, max_tokens=3 * 256).engine.generate(prompts, n_new, sp, stop, batch_size=3)
    assert "stop" in finish and "length" in finish
    for i, (p, got) in enumerate(zip(prompts, toks)):
        state, seq = stream_state(sp.seed, i), list(p)
        for k, t in enumerate(got):
            lg = plain_logits(seq)[-1]
            want, state = SP.sample(lg, sp.temperature, sp.top_k, sp.top_p, sp.min_p, state)
            assert want == t, f"request {i} token {k}: library {t}, plain sampler {want}"
            seq.append(t)
        assert finish[i] == ("stop" if got[-1] in stop else "length") and (got[-1] in stop or len(got) == n_new)
        assert not any(t in stop for t in got[:-1])
    if sp.greedy:
        model = load_model(d, dtype="bfloat16")
        toks, _ = Session(model, max_tokens=3 * 256).engine.generate(prompts, n_new, sp, [], batch_size=3)
        for i, (p, got) in enumerate(zip(prompts, toks)):
            ref = plain_logits(list(p) + got)
            for k, t in enumerate(got):
                row = ref[len(p) - 1 + k]
                assert row[t] >= row.max() - 2 * tolerance("bfloat16", ref, tiny.spread_of("E")), (i, k, t)


def test_prompts_beyond_the_budget_of_a_step_go_in_as_several_steps(folders):
    """Both loops cut a batch of long prompts into steps of at most so many tokens, each appending to
    what the slots hold; they cut alike, so their tokens are the same, and in 32-bit they are the
    tokens of the uncut batch."""
    from picolm_amd import SamplingParams, generate
    from picolm_amd.engine import Session, load_model
    from picolm_amd.generation import prefill_steps
    d = folders["D"]
    V = tiny.TINY_D["vocab_size"]
    model = load_model(d, dtype="float32")
    rng = np.random.default_rng(43)
    lens = (300, 7, 130, 64, 65)
    prompts = [tiny.random_tokens(rng, n, V) for n in lens]
    steps = prefill_steps(lens, 128)
    assert len(steps) > 3 and all(sum(c for _, _, c in st) <= 5 * 64 for st in steps)
    assert sorted((i, f, c) for st in steps for i, f, c in st if f == 0) == [(i, 0, min(n, 64)) for i, n in enumerate(lens)]
    for sp in (SamplingParams(), SamplingParams(0.9, 20, 0.95, 0.0, 3)):
        whole = generate(Session(model, max_tokens=2048), prompts, 12, sp, stop_ids=[])
        cut = generate(Session(model, max_tokens=2048), prompts, 12, sp, stop_ids=[], prefill_step_tokens=128)
        toks, _ = Session(model, max_tokens=2048).engine.generate(prompts, 12, sp, [], prefill_step_tokens=128)
        assert toks == [r.tokens for r in cut]
        if sp.greedy:
            assert toks == [r.tokens for r in whole]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_a_client_written_in_c_builds_a_program_by_hand_and_steps_it(dtype):
    """tests/c_client/tiny_llama.c sees the library through engine.h and api.h alone (compiled as
    C11): it writes the launch program of a two-layer Llama by hand, steps unequal prompts and
    single tokens, lets the library's loop generate, and holds the logits against a plain forward
    pass of its own in double precision.  It exits with 0 when all of that agrees."""
    import os
    import subprocess
    from c_client import build as c_client
    from picolm_amd import kernels
    library = kernels.lib()._name
    exe = c_client.binary(library)
    env = dict(os.environ, LD_LIBRARY_PATH=os.pathsep.join([os.path.dirname(library), os.environ.get("LD_LIBRARY_PATH", "")]))
    out = subprocess.run([exe, dtype], env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    assert out.stdout.startswith(f"ok {dtype}: worst difference of the logits"), out.stdout
    print(out.stdout.strip())
