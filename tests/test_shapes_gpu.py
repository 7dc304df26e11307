"""Logits at the layer sizes that the benchmark times, with seeded random weights made on the GPU:
the shapes of bench.py (Llama-3.1-8B, Llama-2-7B, Llama-3.1-70B, Llama-3.2-1B, and one with heads of
96) at one or two layers, and the Llama-3.1-8B shape at its full depth of 32 layers.

The kernels that only such sizes reach are checked here in the model: 256x256 prefill tiles, a
head of 128,256 rows (tied to the embedding in the 1B shape), tiles of 128 weight rows for up to
16 activation rows, skinny products staged through LDS with K of 11,008 to 28,672, 320-column
tiles for a qkv product of 10,240 rows, one query head per KV head in the decode attention (7B),
head size 64 at a width of 2,048 (1B), and a head size that is no power of two (96) on the matrix
cores.  The bfloat16 engine is held to the 32-bit engine under
every cutting of the work, and the 32-bit engine to the plain implementation on a short request.
picolm checks its fast path against its plain one in the same way (picolm/picolm.c:1437-1463,
warning above 1e-2; :1592-1604)."""
import gc

import numpy as np
import pytest
import torch

import tiny
from bench import SHAPES as BENCH_SHAPES
from plain import llama_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SEED = 8
# (layers, context the rotary tables are laid out for)
LAYERS = {"llama31-8b": 2, "llama2-7b": 2, "llama31-70b": 1, "llama32-1b": 2, "heads96": 2}


def shape_config(name: str, layers: int) -> dict:
    c = dict(BENCH_SHAPES[name]["config"], num_hidden_layers=layers, max_position_embeddings=4096, rope_style="half")
    return c


def spread_of(name: str) -> float:
    return tiny.spread(BENCH_SHAPES[name]["config"]["hidden_size"], BENCH_SHAPES[name]["std"])


def make_models(name: str, layers: int):
    from picolm_amd import LlamaConfig
    from picolm_amd.engine import random_model
    cfg = LlamaConfig.from_dict(shape_config(name, layers))
    # the same bfloat16 values in both: the 32-bit runtime widens them exactly
    return {dt: random_model(cfg, seed=SEED, std=BENCH_SHAPES[name]["std"], dtype=dt, device=DEV) for dt in ("float32", "bfloat16")}


@pytest.fixture(scope="module", params=sorted(LAYERS))
def shaped(request):
    name = request.param
    models = make_models(name, LAYERS[name])
    yield name, models
    models.clear()
    gc.collect()
    torch.cuda.empty_cache()


class LazyWeights:
    """The model's weights as float64 arrays on the host, each made again from the same seed when
    it is asked for (bfloat16 values, widened exactly), so that a model of any depth needs no
    second copy in host memory."""

    def __init__(self, model, std):
        self.specs = {s.name: s for s in model.tensor_specs() if s.init is not None}
        self.std = std

    def __getitem__(self, name):
        from picolm_amd.weights import random_tensor
        return random_tensor(self.specs[name], SEED, self.std, 0.0, torch.bfloat16, DEV).float().cpu().double().numpy()

    def get(self, name, default=None):
        return self[name] if name in self.specs else default


def engine_against_plain(name, models, layers, n_prompt, n_decode):
    from picolm_amd.engine import Session
    c = shape_config(name, layers)
    rng = np.random.default_rng(80)
    toks = tiny.random_tokens(rng, n_prompt + n_decode, c["vocab_size"])
    ref = P.forward(LazyWeights(models["float32"], BENCH_SHAPES[name]["std"]), c, toks)
    s = Session(models["float32"], max_tokens=64)
    [a] = s.begin(1)
    got = s.step([a], [toks[:n_prompt]], [list(range(n_prompt))]).double().cpu().numpy()
    rest = np.concatenate([s.step([a], [[t]]).double().cpu().numpy() for t in toks[n_prompt:]])
    err = max(np.abs(got - ref[:n_prompt]).max(), np.abs(rest - ref[n_prompt:]).max())
    return err, ref


def bfloat16_against_32_bit(name, models, lens, bound):
    """The bfloat16 engine against the 32-bit engine (each request whole) under the three cuttings:
    whole, the last 32 tokens one by one, and two unequal batches one after the other in the same
    slots.  `bound(ref)`: the largest distance accepted.  Returns the worst distance as a share of
    the bound, per cutting."""
    from picolm_amd.engine import Session
    V = BENCH_SHAPES[name]["config"]["vocab_size"]
    rng = np.random.default_rng(81)
    reqs = [tiny.random_tokens(rng, n, V) for n in lens]
    f32 = Session(models["float32"], max_tokens=1024)
    truth = []
    for r in reqs:                                          # the 32-bit engine, each request whole
        [a] = f32.begin(1)
        truth.append(f32.step([a], [r], [list(range(len(r)))]).double().cpu().numpy())
        f32.release([a])
    del f32
    one_batch = sum((len(r) + 63) // 64 for r in reqs[3:]) * 64
    s = Session(models["bfloat16"], max_tokens=one_batch, n_slots=3)
    worst = {"whole": 0.0, "tail": 0.0, "batches": 0.0}

    def check(got, ref, cutting, what):
        err = float(np.abs(got.double().cpu().numpy() - ref).max())
        worst[cutting] = max(worst[cutting], err / bound(ref))
        assert err <= bound(ref), (name, cutting, what, err, bound(ref))
    for i, r in enumerate(reqs):                            # whole
        [a] = s.begin(1)
        check(s.step([a], [r], [list(range(len(r)))]), truth[i], "whole", i)
        s.release([a])
    for i, r in enumerate(reqs):                            # the last 32 tokens one by one
        [a] = s.begin(1)
        n0 = len(r) - 32
        check(s.step([a], [r[:n0]]), truth[i][n0 - 1:n0], "tail", f"{i} prompt")
        for j in range(n0, len(r)):
            check(s.step([a], [[r[j]]]), truth[i][j:j + 1], "tail", f"{i} position {j}")
        s.release([a])
    for ids in ([0, 1, 2], [3, 4, 5]):                      # unequal batches, one after the other in the same slots
        n_dec = dict(zip(ids, (3, 9, 20)))
        pos = {i: len(reqs[i]) - n_dec[i] for i in ids}
        slots = dict(zip(ids, s.begin(3)))
        got = s.step([slots[i] for i in ids], [reqs[i][:pos[i]] for i in ids])
        for k, i in enumerate(ids):
            check(got[k:k + 1], truth[i][pos[i] - 1:pos[i]], "batches", f"prompt {i}")
        live = list(ids)
        while live:
            got = s.step([slots[i] for i in live], [[reqs[i][pos[i]]] for i in live])
            for k, i in enumerate(live):
                check(got[k:k + 1], truth[i][pos[i]:pos[i] + 1], "batches", f"decode {i} at {pos[i]}")
                pos[i] += 1
            for i in [i for i in live if pos[i] == len(reqs[i])]:
                s.release([slots[i]])
                live.remove(i)
    assert s.recorded_steps() >= 2
    return worst


def test_the_32_bit_engine_against_the_plain_implementation(shaped):
    name, models = shaped
    err, ref = engine_against_plain(name, models, LAYERS[name], 17, 7)
    bound = tiny.tolerance("float32", ref, spread_of(name), LAYERS[name])
    print(f"{name}, {LAYERS[name]} layers, 32-bit engine against the plain implementation: {err:.3e} (bound {bound:.3e})")
    assert err <= bound


def test_bfloat16_against_32_bit_under_every_cutting(shaped):
    name, models = shaped
    worst = bfloat16_against_32_bit(name, models, (33, 70, 64, 129, 200, 320),
                                    lambda ref: tiny.tolerance("bfloat16", ref, spread_of(name), LAYERS[name]))
    print(f"{name}, {LAYERS[name]} layers, bfloat16 against 32-bit, worst share of the bound: " +
          ", ".join(f"{k} {v:.3f}" for k, v in worst.items()))


def test_full_depth_of_the_8b_shape():
    """All 32 layers of the Llama-3.1-8B shape: the 32-bit engine against the plain implementation
    on a short request, and the bfloat16 engine against the 32-bit engine under every cutting."""
    name, layers = "llama31-8b", BENCH_SHAPES["llama31-8b"]["config"]["num_hidden_layers"]
    models = make_models(name, layers)
    try:
        err, ref = engine_against_plain(name, models, layers, 9, 3)
        bound = tiny.tolerance("float32", ref, spread_of(name), layers)
        print(f"{name}, {layers} layers, 32-bit engine against the plain implementation: {err:.3e} (bound {bound:.3e})")
        assert err <= bound
        worst = bfloat16_against_32_bit(name, models, (33, 40, 64, 70, 97, 130),
                                        lambda r: tiny.tolerance("bfloat16", r, spread_of(name), layers))
        print(f"{name}, {layers} layers, bfloat16 against 32-bit, worst share of the bound: " +
              ", ".join(f"{k} {v:.3f}" for k, v in worst.items()))
    finally:
        models.clear()
        gc.collect()
        torch.cuda.empty_cache()


def test_sixty_four_prompts_in_one_step():
    """The prompts of a batch of 64 as the generation loop issues them: in one step if they fit the
    step's token budget, else in the steps that `prefill_steps` cuts.  The last row of some of them
    against the same prompt alone; then decode steps of all 64 (tiles of 64 rows, cut along K)."""
    from picolm_amd.engine import Session
    from picolm_amd.generation import SessionStepper
    name = "llama31-8b"
    models = make_models(name, 2)
    del models["float32"]
    SPREAD = spread_of(name)
    V = BENCH_SHAPES[name]["config"]["vocab_size"]
    rng = np.random.default_rng(82)
    lens = [int(x) for x in rng.integers(128, 1200, size=64)]
    prompts = [tiny.random_tokens(rng, n, V) for n in lens]
    pages = sum((n + 70) // 64 for n in lens)
    s = Session(models["bfloat16"], max_tokens=pages * 64, n_slots=64)
    slots = s.begin(64)
    stepper = SessionStepper(s)
    assert sum(lens) > stepper.prefill_step_tokens          # more than one step
    together = stepper.step(slots, prompts).clone()
    alone = Session(models["bfloat16"], max_tokens=2048)
    picks = [0, 17, 40, 63, int(np.argmax(lens)), int(np.argmin(lens))]
    for i in picks:
        [a] = alone.begin(1)
        ref = alone.step([a], [prompts[i]]).double().cpu().numpy()
        alone.release([a])
        err = np.abs(together[i:i + 1].double().cpu().numpy() - ref).max()
        assert err <= tiny.tolerance("bfloat16", ref, SPREAD), (i, lens[i], err)
    # three decode steps of the 64, against each of the picked sequences alone
    nxt = [[int(t)] for t in together.argmax(dim=1).tolist()]
    cont = {i: [nxt[i][0]] for i in picks}
    for _ in range(3):
        logits = s.step(slots, nxt)
        for i in picks:
            [a] = alone.begin(1)
            ref = alone.step([a], [prompts[i] + cont[i]]).double().cpu().numpy()
            alone.release([a])
            err = np.abs(logits[i:i + 1].double().cpu().numpy() - ref).max()
            assert err <= tiny.tolerance("bfloat16", ref, SPREAD), ("decode", i, err)
        nxt = [[int(t)] for t in logits.argmax(dim=1).tolist()]
        for i in picks:
            cont[i].append(nxt[i][0])
