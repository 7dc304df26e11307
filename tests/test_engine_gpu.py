"""The engine against the plain implementation on the GPU, in 32-bit and in bfloat16, under
every way of cutting the work: each request whole; its last 32 tokens one by one; batches of
unequal lengths whose shorter requests end earlier, one batch after another in a cache that
only holds one batch, so that slots and pages are used again.  The first three go through
bin/trace_run as a subprocess, the rest through the library in this process."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import tiny
from plain import llama_plain as P
from plain import sampler_plain as SP
from replay_util import ROOT, TraceRun

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

LENGTHS = {"A": [33, 47, 64, 65, 100, 128], "B": [33, 40, 64, 129, 200, 256], "C": [34, 63, 65, 128, 190, 300],
           "D": [33, 50, 64, 127, 130, 260], "E": [33, 64, 70, 129, 200, 320], "F": [33, 45, 64, 66, 131, 250],
           "G": [33, 64, 65, 130, 300, 700]}


tolerance = tiny.tolerance      # 2e-5 / 2e-2 of the largest logit, wider by sqrt(spread) for weights of a spread above 1


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("models")
    return {w: tiny.make_model_dir(tmp, w) for w in tiny.CONFIGS}


@pytest.fixture(scope="module")
def requests_and_truth(folders):
    out = {}
    for w, d in folders.items():
        V = tiny.read_config(d)["vocab_size"]
        rng = np.random.default_rng(ord(w))
        reqs = [tiny.random_tokens(rng, n, V) for n in LENGTHS[w]]
        out[w] = (reqs, [tiny.plain_logits(d, r) for r in reqs])
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E", "F", "G"])
def test_replay_whole_tail_and_batches(which, dtype, folders, requests_and_truth, tmp_path):
    reqs, truth = requests_and_truth[which]
    one_batch = sum((len(r) + 63) // 64 for r in reqs[3:]) * 64          # room for the larger batch only
    tr = TraceRun(folders[which], dtype, str(tmp_path / "out"), one_batch)
    worst = 0.0

    def check(got, ref, what):
        nonlocal worst
        err = float(np.abs(got.astype(np.float64) - ref).max())
        worst = max(worst, err)
        assert err <= tolerance(dtype, ref), f"{which} {dtype} {what}: {err}"
    # 1. each request alone and whole, every position wanted
    for i, r in enumerate(reqs):
        got = tr.step([(f"w{i}", r, range(len(r)))], end=[f"w{i}"])
        check(got, truth[i], f"whole request {i}")
    # 2. each request alone, the last 32 tokens one by one
    for i, r in enumerate(reqs):
        n0 = len(r) - 32
        got = tr.step([(f"t{i}", r[:n0], [n0 - 1])])
        check(got, truth[i][n0 - 1:n0], f"tail request {i} prompt")
        for j in range(n0, len(r)):
            got = tr.step([(f"t{i}", [r[j]], [0])], end=[f"t{i}"] if j == len(r) - 1 else [])
            check(got, truth[i][j:j + 1], f"tail request {i} position {j}")
    # 3. two batches of unequal lengths, one after the other; requests decode 3, 9, 20 tokens
    for ids in ([0, 1, 2], [3, 4, 5]):
        n_dec = dict(zip(ids, (3, 9, 20)))
        pos = {i: len(reqs[i]) - n_dec[i] for i in ids}
        got = tr.step([(f"b{i}", reqs[i][:pos[i]], [0, pos[i] - 1]) for i in ids])
        for k, i in enumerate(ids):
            check(got[2 * k:2 * k + 2], truth[i][[0, pos[i] - 1]], f"batch prompt of request {i}")
        live = list(ids)
        while live:
            ending = [i for i in live if pos[i] == len(reqs[i]) - 1]
            got = tr.step([(f"b{i}", [reqs[i][pos[i]]], [0]) for i in live], end=[f"b{i}" for i in ending])
            for k, i in enumerate(live):
                check(got[k:k + 1], truth[i][pos[i]:pos[i] + 1], f"batch decode of request {i} at {pos[i]}")
                pos[i] += 1
            live = [i for i in live if i not in ending]
    # a step that wants nothing writes nothing
    assert tr.step([("z", reqs[0][:5], [])], end=["z"]) is None
    tr.close()
    print(f"{which} {dtype}: worst error {worst:.3e}")


def test_replay_reports_a_full_cache(folders, tmp_path):
    tr = TraceRun(folders["A"], "float32", str(tmp_path / "o"), 64)
    assert tr.step([("a", [1] * 60, [59])]).shape == (1, 256)
    with pytest.raises(RuntimeError):
        tr.step([("b", [1] * 10, [0])])          # no page left: the program stops with an error
    assert tr.proc.wait(timeout=60) != 0


# -------------------------------------------------------------------------------------------
def session(folder, dtype, max_tokens=2048, **kw):
    from picolm_amd.engine import Session, load_model
    return Session(load_model(folder, dtype=dtype), max_tokens=max_tokens, **kw)


_WIDE_TRUTH = {}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which,n_seq", [("E", 20), ("E", 64), ("D", 33), ("E", 100), ("D", 300)])
def test_a_wide_batch_decodes_like_its_sequences_alone(which, n_seq, dtype, folders):
    """Decode batches of 17 to 64 sequences take kernels of their own (tiles of 64 rows cut along
    K, the norm split between the products where the widths allow), and more than 64 the prefill's
    (300 sequences: several rows of tiles).
    Unequal prompts, six steps, every sequence's logits against the plain implementation of that
    sequence alone."""
    d = folders[which]
    V = tiny.read_config(d)["vocab_size"]
    rng = np.random.default_rng(n_seq)
    lens = [int(x) for x in rng.integers(3, 90, size=n_seq)]
    n_dec = 6
    seqs = [tiny.random_tokens(rng, n + n_dec, V) for n in lens]
    if (which, n_seq) not in _WIDE_TRUTH:           # (the same for both precisions)
        _WIDE_TRUTH[(which, n_seq)] = [tiny.plain_logits(d, q) for q in seqs]
    truth = _WIDE_TRUTH[(which, n_seq)]
    s = session(d, dtype, max_tokens=n_seq * 192, n_slots=n_seq)
    slots = s.begin(n_seq)
    got = s.step(slots, [q[:n] for q, n in zip(seqs, lens)]).double().cpu().numpy()
    for i, n in enumerate(lens):
        assert np.abs(got[i] - truth[i][n - 1]).max() <= tolerance(dtype, truth[i]), ("prompt", i)
    for j in range(n_dec):
        got = s.step(slots, [[q[n + j]] for q, n in zip(seqs, lens)]).double().cpu().numpy()
        for i, n in enumerate(lens):
            err = np.abs(got[i] - truth[i][n + j]).max()
            assert err <= tolerance(dtype, truth[i]), (which, dtype, "step", j, "sequence", i, err)
    s.release(slots)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["B", "E"])
def test_single_token_steps_that_do_not_want_every_row(which, dtype, folders):
    """Steps of one token per sequence in which one sequence wants nothing, another its one row and
    a third the same row twice: such a step is planned like a prefill step with a gather of the
    wanted rows, not as the decode step that replays a recording.  They alternate with plain decode
    steps of the same batch, before and after that batch size's recording exists; every row against
    the plain implementation."""
    d = folders[which]
    V = tiny.read_config(d)["vocab_size"]
    rng = np.random.default_rng(17)
    lens, n_dec = [70, 5, 33], 12
    seqs = [tiny.random_tokens(rng, n + n_dec, V) for n in lens]
    truth = [tiny.plain_logits(d, q) for q in seqs]
    s = session(d, dtype, max_tokens=1024, n_slots=3)
    slots = s.begin(3)
    s.step(slots, [q[:n] for q, n in zip(seqs, lens)], [[], [], []])
    wants = [None, [[], [0], [0, 0]], None, None, [[0], [], []], [[], [], [0]], None, [[], [], []], [[0], [0], [0]], None,
             [[0, 0], [], [0]], None]
    recorded_before = s.recorded_steps()
    for j, want in enumerate(wants):
        got = s.step(slots, [[q[n + j]] for q, n in zip(seqs, lens)], want)
        rows = [i for i in range(3) for _ in (want[i] if want is not None else [0])]
        assert got.shape[0] == len(rows)
        got = got.double().cpu().numpy()
        for k, i in enumerate(rows):
            err = np.abs(got[k] - truth[i][lens[i] + j]).max()
            assert err <= tolerance(dtype, truth[i], tiny.spread_of(which)), (which, dtype, "step", j, "sequence", i, err)
    assert recorded_before == 0 and s.recorded_steps() == 1     # the plain decode steps were recorded meanwhile
    s.release(slots)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_first_tokens(dtype, folders):
    d = folders["C"]
    rng = np.random.default_rng(11)
    toks = tiny.random_tokens(rng, 400, tiny.TINY_C["vocab_size"])
    ref = tiny.plain_logits(d, toks)
    s = session(d, dtype)
    [a] = s.begin(1)
    for j, t in enumerate(toks):                 # a prompt of one token, then 399 single steps
        got = s.step([a], [[t]]).double().cpu().numpy()
        err = np.abs(got[0] - ref[j]).max()
        assert err <= tolerance(dtype, ref), (j, err)
    assert s.length(a) == 400


def test_decoding_at_contexts_of_thousands_of_tokens(tmp_path):
    """Twelve sequences of about 5,000 tokens: enough pages for the decode attention to take chunks
    of 64 (and, when most sequences have ended, 32 and 16), each sequence several chunks whose
    partial results are merged.  All twelve are beginnings of one token sequence, so that one pass
    of the plain implementation knows every logit; they differ in length, slot and pages."""
    from picolm_amd import LlamaConfig, write_random_model
    from picolm_amd.engine import Session, load_model
    cfg = dict(architectures=["LlamaForCausalLM"], hidden_size=256, intermediate_size=344, num_attention_heads=8,
               num_key_value_heads=8, num_hidden_layers=1, vocab_size=300, head_dim=32, rms_norm_eps=1e-5, rope_theta=10000.0,
               tie_word_embeddings=False, max_position_embeddings=8192, torch_dtype="bfloat16")
    d = write_random_model(LlamaConfig.from_dict(cfg), str(tmp_path / "long"), seed=21, std=0.05)
    rng = np.random.default_rng(21)
    toks = tiny.random_tokens(rng, 5010, 300)
    truth = tiny.plain_logits(d, toks)
    lens = [5000 - 37 * i for i in range(12)]
    s = Session(load_model(d, dtype="bfloat16"), max_tokens=12 * 5120)
    slots = s.begin(12)
    got = s.step(slots, [toks[:n] for n in lens]).double().cpu().numpy()          # the prompts, all in one step
    tol_ = tiny.tolerance("bfloat16", truth, tiny.spread(256, 0.05))
    for i, n in enumerate(lens):
        assert np.abs(got[i] - truth[n - 1]).max() <= tol_, ("prefill", i)
    from plan_reference import decode_pages_per_chunk
    seen = set()
    live = list(range(12))
    for step in range(6):
        if step == 2:
            live = live[:8]                       # fewer sequences: shorter chunks
        if step == 4:
            live = live[:4]
        pos = [lens[i] + step for i in live]
        seen.add(decode_pages_per_chunk(pos, 8, 64))
        got = s.step([slots[i] for i in live], [[toks[lens[i] + step]] for i in live]).double().cpu().numpy()
        for k, i in enumerate(live):
            assert np.abs(got[k] - truth[lens[i] + step]).max() <= tol_, (step, i)
    assert seen == {64, 32, 16}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_stale_cache_contents_change_nothing(dtype, folders):
    d = folders["B"]
    rng = np.random.default_rng(12)
    V = tiny.TINY_B["vocab_size"]
    s = session(d, dtype, max_tokens=256)
    for g in s.cache.kv:                         # whatever a freed slot leaves behind must not matter
        g.k.fill_(float("nan"))
        g.v.fill_(float("nan"))
    for n in (70, 3, 129):
        toks = tiny.random_tokens(rng, n, V)
        ref = tiny.plain_logits(d, toks)
        [a] = s.begin(1)
        got = s.step([a], [toks[:-1]], [list(range(n - 1))]).double().cpu().numpy() if n > 1 else None
        last = s.step([a], [[toks[-1]]]).double().cpu().numpy()
        s.release([a])
        assert np.abs(got - ref[:-1]).max() <= tolerance(dtype, ref)
        assert np.abs(last[0] - ref[-1]).max() <= tolerance(dtype, ref)


def test_padding_free_batch_equals_each_alone_bitwise_in_f32(folders):
    """What else is in the batch may change a result by rounding only; with the float kernels,
    whose summation order per row does not depend on the batch, not at all."""
    d = folders["A"]
    rng = np.random.default_rng(13)
    prompts = [tiny.random_tokens(rng, n, 256) for n in (5, 11, 17)]
    s = session(d, "float32")
    alone = []
    for p in prompts:
        [a] = s.begin(1)
        alone.append(s.step([a], [p]).clone())
        s.release([a])
    slots = s.begin(3)
    together = s.step(slots, prompts)
    for i in range(3):
        assert torch.equal(together[i], alone[i][0])


def test_step_errors(folders):
    from picolm_amd.cache import CacheFull
    from picolm_amd.engine import StepError
    s = session(folders["A"], "float32", max_tokens=128)
    [a] = s.begin(1)
    with pytest.raises(StepError, match="vocabulary"):
        s.step([a], [[1, 256]])
    with pytest.raises(StepError, match="not live"):
        s.step([5], [[1]])
    with pytest.raises(StepError, match="twice"):
        s.step([a, a], [[1], [2]])
    with pytest.raises(CacheFull):
        s.step([a], [[1] * 129])                 # longer than max_position_embeddings / the cache
    assert s.length(a) == 0                      # a refused step leaves the sequence where it was
    s.step([a], [[1] * 128])
    with pytest.raises(CacheFull):
        s.step([a], [[1]])


# ------------------------------------------------------------------------------------------- generation
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(dtype, folders):
    from picolm_amd.engine import load_model
    from picolm_amd.generation import generate
    d = folders["A"]
    rng = np.random.default_rng(0)
    prompts = [tiny.random_tokens(rng, n, 256) for n in (5, 11, 17)]       # three prompts of unequal length, 8 greedy steps
    model = load_model(d, dtype=dtype)
    got = generate(model, prompts, max_new_tokens=8, stop_ids=())
    for p, r in zip(prompts, got):
        seq = list(p)
        for k in range(8):
            lg = tiny.plain_logits(d, seq)[-1]
            top2 = np.sort(lg)[-2:]
            if top2[1] - top2[0] < 2 * tolerance(dtype, lg):
                break                              # a near tie: either choice is right
            assert r.tokens[k] == int(np.argmax(lg)), (k, r.tokens)
            seq.append(r.tokens[k])
        assert len(r.tokens) == 8 and r.finish == "length"
    # the entry point takes the model's folder as well, as picolm's takes a file name
    import picolm_amd
    again = picolm_amd.generate(d, prompts, max_new_tokens=8, stop_ids=(), dtype=dtype)
    assert [r.tokens for r in again] == [r.tokens for r in got]


def test_temperature_generation_follows_the_plain_sampler(folders):
    """Tiny B's workload: prompts of 1/9/30/64 tokens, 12 steps at temperature 0.8, fixed seed.
    Each sampled token must be what the plain sampler draws from the plain logits of the
    engine's own sequence so far, with that request's generator stream."""
    from picolm_amd.engine import load_model
    from picolm_amd.generation import generate
    from picolm_amd.sampling import SamplingParams, stream_state
    d = folders["B"]
    rng = np.random.default_rng(1)
    prompts = [tiny.random_tokens(rng, n, 384) for n in (1, 9, 30, 64)]
    model = load_model(d, dtype="float32")
    for batch_size in (4, 3):                     # the streams do not depend on the batching
        got = generate(model, prompts, max_new_tokens=12, params=SamplingParams(temperature=0.8, seed=5), stop_ids=(),
                       batch_size=batch_size)
        for i, (p, r) in enumerate(zip(prompts, got)):
            state = stream_state(5, i)
            seq = list(p)
            for k in range(12):
                lg = tiny.plain_logits(d, seq)[-1]
                want, state = SP.sample(lg, 0.8, 0, 1.0, 0.0, state)
                assert want == r.tokens[k], f"request {i} token {k}: engine {r.tokens[k]} plain {want}"
                seq.append(want)


def test_stop_tokens_end_sequences_early(folders):
    from picolm_amd.engine import load_model
    from picolm_amd.generation import generate
    d = folders["A"]
    model = load_model(d, dtype="float32")
    rng = np.random.default_rng(2)
    prompts = [tiny.random_tokens(rng, n, 256) for n in (4, 9, 15, 6)]
    free = generate(model, prompts, max_new_tokens=10, stop_ids=())
    stop = free[1].tokens[3]                      # make request 1 stop at its fourth token
    got = generate(model, prompts, max_new_tokens=10, stop_ids=[stop], batch_size=2)
    for f, g in zip(free, got):
        if stop in f.tokens:
            cut = f.tokens.index(stop) + 1
            assert g.tokens == f.tokens[:cut] and g.finish == "stop"
        else:
            assert g.tokens == f.tokens and g.finish == "length"
    assert got[1].finish == "stop" and len(got[1].tokens) <= 4


def test_command_line(folders, tmp_path):
    d = folders["A"]
    env = dict(os.environ, PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "picolm"), d, "-p", "5 17, 3", "-n", "6", "-t", "0",
                        "--dtype", "float32"], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0, r.stderr
    toks = [int(t) for t in r.stdout.split()]
    seq = [5, 17, 3]
    for t in toks:
        if t == 2:                                 # the configuration's stop token
            break
        assert t == int(np.argmax(tiny.plain_logits(d, seq)[-1]))
        seq.append(t)
    assert len(toks) <= 6 and "Prefill: 3 tokens" in r.stderr and "Generation:" in r.stderr
    # several prompts from standard input make a batch; a seed makes sampling repeatable
    cmd = [sys.executable, "-m", "picolm_amd", d, "-n", "5", "-s", "7", "--dtype", "float32", "--json"]
    a = subprocess.run(cmd, input="1 2 3\n9 8\n", capture_output=True, text=True, env=env, timeout=300, cwd=ROOT)
    b = subprocess.run(cmd, input="1 2 3\n9 8\n", capture_output=True, text=True, env=env, timeout=300, cwd=ROOT)
    assert a.returncode == 0 and a.stdout == b.stdout or json.loads(a.stdout)["tokens"] == json.loads(b.stdout)["tokens"]
    assert len(json.loads(a.stdout)["tokens"]) == 2
    # the random-weights mode writes a folder that loads
    cfg = tmp_path / "c.json"
    cfg.write_text(json.dumps(tiny.TINY_C))
    w = subprocess.run([sys.executable, "-m", "picolm_amd", "--random-model", str(tmp_path / "m"), "--config", str(cfg),
                        "-s", "3"], capture_output=True, text=True, env=env, timeout=300, cwd=ROOT)
    assert w.returncode == 0, w.stderr
    ls = subprocess.run([sys.executable, "-m", "picolm_amd", str(tmp_path / "m"), "--list-tensors"], capture_output=True,
                        text=True, env=env, timeout=300, cwd=ROOT)
    assert "model.layers.0.self_attn.q_proj.weight\t[96, 80]\tbfloat16" in ls.stdout


def test_command_line_checks_and_speed_runs(folders, capsys):
    """picolm's --gpu-diff, --gpu-attn-diff, --benchmark-ctx and --benchmark, run in this process."""
    from picolm_amd import cli
    # products: a decode batch, a wide decode batch, a prompt (three kernels of the matrix-core path)
    for S, I, O in ((8, 512, 1024), (40, 1024, 520), (300, 192, 1031)):
        assert cli.main(["--gpu-diff", str(S), str(I), str(O)]) == 0
    err = capsys.readouterr().err
    assert err.count("PASS") == 3 and "matrix-core kernel against float64" in err
    # attention: a head size of the matrix-core kernels, and one that only the plain kernels take
    assert cli.main(["--gpu-attn-diff", "200", "8", "2", "64"]) == 0
    assert cli.main(["--gpu-attn-diff", "70", "6", "3", "20", "-s", "5"]) == 0
    assert cli.main(["--gpu-attn-diff", "150", "4", "2", "96"]) == 0          # matrix cores at another head size
    assert cli.main(["--gpu-attn-diff", "130", "2", "1", "320"]) == 0         # wider than the 256 columns a tile holds at a time
    with pytest.raises(SystemExit, match="up to 1024"):
        cli.main(["--gpu-attn-diff", "10", "2", "1", "1026"])
    assert capsys.readouterr().err.count("PASS") == 4
    d = folders["A"]
    assert cli.main([d, "--benchmark-ctx", "-p", "5 6 7 8 9", "-n", "11", "-c", "100", "-t", "0"]) == 0
    rows = [l for l in capsys.readouterr().err.splitlines() if l and l[0].isdigit()]
    # 16 tokens a step into a context of 100: steps at 0, 16, ..., 80
    assert [int(r.split(",")[0]) for r in rows] == list(range(0, 96, 16)) and all(float(x) > 0 for r in rows for x in r.split(",")[1:])
    assert cli.main([d, "--benchmark", "--benchmark-iterations", "2", "-p", "5 6 7", "-n", "9", "-t", "0.7"]) == 0
    err = capsys.readouterr().err
    assert "--- Iteration 2" in err and "--- Iteration 3" not in err
    assert err.count("Prefill: 3 tokens") == 2 and err.count("Generation: 9 tokens") == 2


def test_missing_tensor_is_reported_when_loading(folders, tmp_path):
    from safetensors.torch import load_file, save_file
    from picolm_amd import WeightsError
    from picolm_amd.engine import load_model
    d = str(tmp_path / "broken")
    os.makedirs(d)
    w = load_file(os.path.join(folders["A"], "model.safetensors"))
    del w["model.layers.1.mlp.gate_proj.weight"]
    w["model.layers.0.self_attn.v_proj.weight"] = w["model.layers.0.self_attn.v_proj.weight"][:16].contiguous()
    save_file(w, os.path.join(d, "model.safetensors"))
    open(os.path.join(d, "config.json"), "w").write(open(os.path.join(folders["A"], "config.json")).read())
    with pytest.raises(WeightsError) as e:
        load_model(d)
    assert e.value.missing == ["model.layers.1.mlp.gate_proj.weight"]
    assert e.value.wrong_shape == [("model.layers.0.self_attn.v_proj.weight", (32, 64), (16, 64))]


def test_recorded_decode_steps_equal_eager_ones(folders):
    """Decode steps replay a recorded HIP graph from their third use on; every replay must give
    what the same step gives when its kernels are launched one by one, with the program's own
    other work (prefills of other requests, releases) between the replays."""
    from picolm_amd.engine import Session, load_model
    d = folders["C"]
    model = load_model(d, dtype="bfloat16")
    rng = np.random.default_rng(21)
    V = tiny.TINY_C["vocab_size"]
    prompts = [tiny.random_tokens(rng, n, V) for n in (70, 5, 33)]
    cont = [tiny.random_tokens(rng, 40, V) for _ in prompts]
    outs = {}
    for graphs in (True, False):
        s = Session(model, max_tokens=1024, graphs=graphs)
        slots = s.begin(3)
        s.step(slots, prompts)
        rows = []
        for j in range(40):
            rows.append(s.step(slots, [[c[j]] for c in cont]).clone())
            if j % 7 == 3:                        # unrelated work between replays
                [x] = s.begin(1)
                s.step([x], [tiny.random_tokens(rng, 90, V)])
                s.release([x])
        outs[graphs] = torch.stack(rows)
        assert (s.recorded_steps() > 0) == graphs
    assert torch.equal(outs[True], outs[False])


def test_more_shapes_of_recorded_decode_steps_than_the_engine_keeps(folders):
    """Batches of 1 to 56 sequences, three decode steps each: every batch size is a recorded step
    of its own, the engine keeps 48 of them and lets the least recently used go.  Each step gives
    the same bits as in a session that launches its kernels one by one, also the shapes that come
    back after they were dropped."""
    from picolm_amd.engine import Session, load_model
    d = folders["A"]
    model = load_model(d, dtype="bfloat16")
    V = tiny.TINY_A["vocab_size"]
    rng = np.random.default_rng(48)
    n_all = 56
    prompts = [tiny.random_tokens(rng, 3 + i % 7, V) for i in range(n_all)]
    order = list(range(1, n_all + 1)) + [1, 2, 3, 56, 30]
    feed = [[tiny.random_tokens(rng, n, V) for _ in range(3)] for n in order]
    outs = {}
    for graphs in (True, False):
        s = Session(model, max_tokens=64 * 2 * n_all, max_seq_len=128, n_slots=n_all, graphs=graphs)
        slots = s.begin(n_all)
        s.step(slots, prompts)
        rows, start = [], 0
        for n, toks in zip(order, feed):
            batch = [slots[(start + k) % n_all] for k in range(n)]      # in turn, so that no sequence outgrows the cache
            start += n
            for t in toks:
                rows.append(s.step(batch, [[x] for x in t]).clone())
        outs[graphs] = rows
        if graphs:
            assert s.recorded_steps() == 48
    for a, b in zip(outs[True], outs[False]):
        assert torch.equal(a, b)


@pytest.mark.parametrize("which", ["C", "D"])
def test_a_batch_that_continues_where_another_stopped(which, folders):
    """One batch ends and gives its slots back; the next gets the same slots (with other pages)
    and its sequences happen to be exactly one token longer than the last ones were.  To the
    recorded decode step that looks like the next step of the old batch; it must not keep what it
    looked up in the page tables for the old one."""
    d = folders[which]
    V = tiny.CONFIGS[which][0]["vocab_size"]
    rng = np.random.default_rng(5)
    s = session(d, "bfloat16", max_tokens=1024)
    hold = s.begin(1)                                   # keeps a page, so that the pages of the second batch differ
    s.step(hold, [tiny.random_tokens(rng, 3, V)])
    first = [tiny.random_tokens(rng, n, V) for n in (40, 70)]
    slots = s.begin(2)
    s.step(slots, [t[:-4] for t in first])
    for j in range(4, 0, -1):                           # decode steps at positions 36..39 and 66..69
        s.step(slots, [[t[-j]] for t in first])
    s.release(slots)
    s.step(hold, [tiny.random_tokens(rng, 130, V)])     # takes pages that the first batch gave back
    second = [tiny.random_tokens(rng, n, V) for n in (41, 71)]
    assert sorted(s.begin(2)) == sorted(slots)
    again = slots                                       # the same slots in the same order as before
    s.step(again, [t[:-1] for t in second])             # prompts of 40 and 70 tokens
    got = s.step(again, [[t[-1]] for t in second]).cpu().numpy()      # decode at positions 40 and 70
    for i, t in enumerate(second):
        ref = tiny.plain_logits(d, t)[-1]
        assert np.abs(got[i] - ref).max() <= tolerance("bfloat16", ref)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_with_tokens_on_the_device_equal_steps_with_tokens_from_the_host(dtype, folders):
    """A decode step may take its tokens from device memory (what the sampler wrote) so that the
    host can hand it over before it has read them.  Several such steps in a row, each launched
    before the one before it has been waited for, across a page boundary and with a sequence
    leaving the batch: the same logits, bit for bit, as steps fed from the host."""
    from picolm_amd.sampling import Sampler, SamplingParams
    d = folders["D"]
    V = tiny.read_config(d)["vocab_size"]
    rng = np.random.default_rng(21)
    prompts = [tiny.random_tokens(rng, n, V) for n in (61, 5, 120)]

    def run(on_device):
        s = session(d, dtype, max_tokens=1024)
        sampler = Sampler(SamplingParams(), 3, DEV)
        slots = s.begin(3)
        logits = s.step(slots, prompts)
        seen, live = [], [0, 1, 2]
        pending = sampler.launch(logits, live)
        for j in range(8):
            if j == 5:                       # the second sequence leaves
                pick, live = [0, 2], [0, 2]
            else:
                pick = None
            if on_device:
                logits = s.step_tokens_on_device([slots[i] for i in live], pending.on_device(pick))
            else:
                toks = pending.wait()
                toks = toks if pick is None else [toks[r] for r in pick]
                logits = s.step([slots[i] for i in live], [[t] for t in toks])
            seen.append(logits.clone())
            pending = sampler.launch(logits, live)
        torch.cuda.synchronize()
        assert [s.length(x) for x in slots] == [61 + 8, 5 + 5, 120 + 8]
        return seen

    a, b = run(True), run(False)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


def test_tokens_on_the_device_are_checked(folders):
    from picolm_amd.engine import StepError
    s = session(folders["A"], "float32")
    slots = s.begin(2)
    s.step(slots, [[1, 2], [3]])
    with pytest.raises(StepError, match="int32"):
        s.step_tokens_on_device(slots, torch.zeros(2, dtype=torch.int64, device=DEV))
    with pytest.raises(StepError, match="int32"):
        s.step_tokens_on_device(slots, torch.zeros(3, dtype=torch.int32, device=DEV))
    s.release([slots[1]])
    with pytest.raises(StepError, match="not live"):
        s.step_tokens_on_device(slots, torch.zeros(2, dtype=torch.int32, device=DEV))


def test_generation_one_step_ahead_equals_generation_step_by_step(folders):
    """The entry point drives a session one step ahead (the next step is launched before this
    step's tokens are read).  With stops, a token limit and several batches in a small cache it
    returns what a loop that reads every step's tokens first returns, with recorded steps and
    without them."""
    from picolm_amd.engine import Session, load_model
    from picolm_amd.generation import GenerationLoop, SessionStepper
    from picolm_amd.sampling import Sampler, SamplingParams
    d = folders["D"]
    V = tiny.read_config(d)["vocab_size"]
    model = load_model(d, dtype="float32")
    rng = np.random.default_rng(31)
    prompts = [tiny.random_tokens(rng, n, V) for n in (3, 70, 20, 64, 9, 33)]
    params = SamplingParams(temperature=0.9, top_k=50, top_p=0.95, seed=5)

    class StepByStep:
        """A stepper without step_ahead: the loop then reads every step's tokens first."""

        def __init__(self, session):
            self._inner = SessionStepper(session)
            self.capacity = self._inner.capacity
            self.begin, self.step, self.release, self.fits = (self._inner.begin, self._inner.step,
                                                              self._inner.release, self._inner.fits)

    def run(stepper_type, graphs, stop_ids):
        s = Session(model, max_tokens=4 * 192, graphs=graphs)
        loop = GenerationLoop(stepper_type(s), lambda n: Sampler(params, n, DEV), stop_ids, batch_size=3)
        out = loop.run(prompts, 40)
        assert s.cache.slots.n_free == s.cache.slots.n_slots
        return [(r.tokens, r.finish) for r in out]

    free = run(SessionStepper, True, ())
    stops = [free[1][0][5], free[4][0][17]]
    want = run(SessionStepper, True, stops)
    assert any(f == "stop" for _, f in want) and any(f == "length" for _, f in want)
    assert run(SessionStepper, False, stops) == want
    assert run(StepByStep, True, stops) == want


# ------------------------------------------------------------------------------------------- further schedules and folders
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["B", "D"])
def test_steps_that_append_several_tokens_to_what_a_slot_holds(which, dtype, folders):
    """A step may bring several tokens for a sequence that already holds some (picolm continues a
    prompt from `start_pos` the same way, picolm/picolm.c:1285-1290, :481-514): alone, next to
    other such sequences, and in one step with sequences that bring a single token.  Every row
    against the plain implementation of the whole sequence."""
    d = folders[which]
    V = tiny.read_config(d)["vocab_size"]
    rng = np.random.default_rng(31)
    seqs = [tiny.random_tokens(rng, n, V) for n in (150, 90, 201)]
    truth = [tiny.plain_logits(d, q) for q in seqs]
    s = session(d, dtype)
    slots = s.begin(3)
    pos = [0, 0, 0]

    def step(cuts, who=(0, 1, 2)):
        got = s.step([slots[i] for i in who], [seqs[i][pos[i]:pos[i] + c] for i, c in zip(who, cuts)],
                     [list(range(c)) for c in cuts]).double().cpu().numpy()
        row = 0
        for i, c in zip(who, cuts):
            err = np.abs(got[row:row + c] - truth[i][pos[i]:pos[i] + c]).max()
            assert err <= tolerance(dtype, truth[i]), (which, dtype, "sequence", i, "from", pos[i], "tokens", c, err)
            row += c
            pos[i] += c
    step([40, 7, 64])                  # the prompts
    step([70, 3, 1])                   # 70 more onto 40 (over a page's end), 3 onto 7, and a single token in the same step
    step([5], who=(0,))                # alone
    step([1, 1, 1])                    # a decode step in between
    step([30, 60, 100])                # and on from there
    step([1, 19], who=(2, 1))          # another order of slots, one token and several
    assert [s.length(x) for x in slots] == pos
    s.release(slots)


@pytest.mark.parametrize("which", ["D", "E"])
def test_a_prefill_step_of_a_thousand_tokens_and_more(which, folders):
    """From 1,024 tokens a step on, the matrix-core path writes no rotated copy of q: the attention
    kernel rotates q itself and a tile-wise kernel writes keys and values.  Prompts that make
    such a step together, one of them continued from what its slot holds; then decode steps, which
    read what that kernel wrote."""
    d = folders[which]
    cfg = tiny.read_config(d)
    rng = np.random.default_rng(77)
    limit = cfg["max_position_embeddings"]
    lens = [min(700, limit - 8), 420]
    while sum(lens) - 37 < 1024:
        lens.append(300)
    n = len(lens)
    seqs = [tiny.random_tokens(rng, m + 4, cfg["vocab_size"]) for m in lens]
    truth = [tiny.plain_logits(d, q) for q in seqs]
    s = session(d, "bfloat16", max_tokens=2048)
    slots = s.begin(n)
    s.step([slots[1]], [seqs[1][:37]])                       # the second prompt's first 37 tokens are held already
    first = [0, 37] + [0] * (n - 2)
    want = [[0, 5, m - f - 1] for m, f in zip(lens, first)]
    got = s.step(slots, [q[f:m] for q, f, m in zip(seqs, first, lens)], want).double().cpu().numpy()
    for i in range(n):
        for k, j in enumerate(want[i]):
            assert np.abs(got[3 * i + k] - truth[i][first[i] + j]).max() <= tolerance("bfloat16", truth[i]), (i, j)
    for j in range(4):
        got = s.step(slots, [[q[m + j]] for q, m in zip(seqs, lens)]).double().cpu().numpy()
        for i in range(n):
            assert np.abs(got[i] - truth[i][lens[i] + j]).max() <= tolerance("bfloat16", truth[i]), (i, "step", j)
    s.release(slots)


@pytest.mark.parametrize("stored", ["float32", "float16"])
def test_folders_stored_in_other_types_than_bfloat16(stored, tmp_path):
    """A folder stored in 32-bit keeps its weights in 32-bit in both runtimes (the bfloat16 runtime
    then multiplies bfloat16 rows by float weights in the float kernel); a float16 folder is
    widened exactly by the 32-bit runtime (picolm keeps float16 as it is, picolm/safetensors.c:163)
    and rounded to bfloat16 by the other."""
    d = tiny.make_model_dir(tmp_path, "B", dtype=stored)
    V = tiny.TINY_B["vocab_size"]
    rng = np.random.default_rng(32)
    toks = tiny.random_tokens(rng, 90, V)
    ref = tiny.plain_logits(d, toks)                       # the plain implementation reads the stored values
    for dtype in ("float32", "bfloat16"):
        s = session(d, dtype, max_tokens=256)
        w = s.model.blocks[0].mixer.qkv.weight
        assert w.dtype == (torch.float32 if stored == "float32" or dtype == "float32" else torch.bfloat16)
        [a] = s.begin(1)
        got = s.step([a], [toks[:60]], [list(range(60))]).double().cpu().numpy()
        rest = np.concatenate([s.step([a], [[t]]).double().cpu().numpy() for t in toks[60:]])
        err = max(np.abs(got - ref[:60]).max(), np.abs(rest - ref[60:]).max())
        # float16 rounded to bfloat16 loses three bits of every weight: the bound of the bfloat16
        # runtime covers it, and the 32-bit runtime must not need it
        assert err <= tolerance(dtype, ref), (stored, dtype, err)


def test_a_longer_session_leaves_an_earlier_sessions_recorded_steps_alone(folders):
    """Both sessions share the model's rotary tables.  The longer one needs more positions; the
    tables that the first one's recorded steps read must stay what and where they were."""
    from picolm_amd.engine import Session, load_model
    d = folders["D"]
    V = tiny.TINY_D["vocab_size"]
    rng = np.random.default_rng(33)
    toks = tiny.random_tokens(rng, 120, V)
    ref = tiny.plain_logits(d, toks)
    model = load_model(d, dtype="bfloat16")
    s1 = Session(model, max_tokens=128)
    [a] = s1.begin(1)
    s1.step([a], [toks[:50]])
    for t in toks[50:60]:
        s1.step([a], [[t]])
    assert s1.recorded_steps() == 1
    s2 = Session(model, max_tokens=512)                    # tables for 512 positions replace those for 128
    junk = [torch.full((1 << 20,), float("nan"), device=DEV) for _ in range(8)]      # whatever was freed is reused
    [b] = s2.begin(1)
    s2.step([b], [toks[:70]])
    for j in range(60, 120):
        got = s1.step([a], [[toks[j]]]).double().cpu().numpy()
        assert np.abs(got[0] - ref[j]).max() <= tolerance("bfloat16", ref), j
    del junk
