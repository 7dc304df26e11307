"""Logits at the layer sizes that the benchmark times: two layers of the Llama-3.1-8B shape
(hidden 4096, 32 heads over 8 KV heads of 128, intermediate 14336, the full vocabulary of 128,256,
llama3 frequency scaling) with seeded random weights N(0, 0.02) made on the GPU.

The kernels that only such sizes reach (256x256 prefill tiles, a head of 128,256 rows, tiles of
128 weight rows for up to 16 activation rows, skinny products staged through LDS with K of 14,336)
are checked here in the model: the bfloat16 engine against the 32-bit engine under every
cutting of the work, and the 32-bit engine against the plain implementation on a short request.
picolm checks its fast path against its plain one in the same way (picolm/picolm.c:1437-1463,
warning above 1e-2)."""
import numpy as np
import pytest
import torch

import tiny
from plain import llama_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
STD = 0.02
SHAPE = dict(
    architectures=["LlamaForCausalLM"], hidden_size=4096, intermediate_size=14336, num_attention_heads=32,
    num_key_value_heads=8, num_hidden_layers=2, vocab_size=128256, head_dim=128, rms_norm_eps=1e-5, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    tie_word_embeddings=False, max_position_embeddings=4096, eos_token_id=2, rope_style="half")
SPREAD = tiny.spread(4096, STD)          # 1.64: the bounds are 1.28 times those of the tiny configurations


@pytest.fixture(scope="module")
def models():
    from picolm_amd import LlamaConfig
    from picolm_amd.engine import random_model
    cfg = LlamaConfig.from_dict(SHAPE)
    # the same bfloat16 values in both: the 32-bit runtime widens them exactly
    return {dt: random_model(cfg, seed=8, std=STD, dtype=dt, device=DEV) for dt in ("float32", "bfloat16")}


def plain_weights(model):
    """The model's weights as float32 arrays on the host, made again from the same seed (bfloat16
    values are exact in float32; NumPy widens them to float64 where the plain functions multiply)."""
    from picolm_amd.weights import random_tensor
    return {s.name: random_tensor(s, 8, STD, 0.0, torch.bfloat16, DEV).float().cpu().numpy()
            for s in model.tensor_specs() if s.init is not None}


def test_the_32_bit_engine_against_the_plain_implementation(models):
    from picolm_amd.engine import Session
    rng = np.random.default_rng(80)
    toks = tiny.random_tokens(rng, 24, SHAPE["vocab_size"])
    ref = P.forward(plain_weights(models["float32"]), SHAPE, toks)
    s = Session(models["float32"], max_tokens=64)
    [a] = s.begin(1)
    got = s.step([a], [toks[:17]], [list(range(17))]).double().cpu().numpy()
    rest = np.concatenate([s.step([a], [[t]]).double().cpu().numpy() for t in toks[17:]])
    err = max(np.abs(got - ref[:17]).max(), np.abs(rest - ref[17:]).max())
    print(f"8B shape, 32-bit engine against the plain implementation: {err:.3e} (bound {tiny.tolerance('float32', ref, SPREAD):.3e})")
    assert err <= tiny.tolerance("float32", ref, SPREAD)


def test_bfloat16_against_32_bit_under_every_cutting(models):
    from picolm_amd.engine import Session
    V = SHAPE["vocab_size"]
    rng = np.random.default_rng(81)
    reqs = [tiny.random_tokens(rng, n, V) for n in (33, 70, 64, 129, 200, 320)]
    f32 = Session(models["float32"], max_tokens=1024)
    truth = []
    for r in reqs:                                          # the 32-bit engine, each request whole
        [a] = f32.begin(1)
        truth.append(f32.step([a], [r], [list(range(len(r)))]).double().cpu().numpy())
        f32.release([a])
    one_batch = sum((len(r) + 63) // 64 for r in reqs[3:]) * 64
    s = Session(models["bfloat16"], max_tokens=one_batch, n_slots=3)
    worst = 0.0

    def check(got, ref, what):
        nonlocal worst
        err = float(np.abs(got.double().cpu().numpy() - ref).max())
        worst = max(worst, err / tiny.tolerance("bfloat16", ref, SPREAD))
        assert err <= tiny.tolerance("bfloat16", ref, SPREAD), (what, err)
    for i, r in enumerate(reqs):                            # whole
        [a] = s.begin(1)
        check(s.step([a], [r], [list(range(len(r)))]), truth[i], f"whole {i}")
        s.release([a])
    for i, r in enumerate(reqs):                            # the last 32 tokens one by one
        [a] = s.begin(1)
        n0 = len(r) - 32
        check(s.step([a], [r[:n0]]), truth[i][n0 - 1:n0], f"tail {i} prompt")
        for j in range(n0, len(r)):
            check(s.step([a], [[r[j]]]), truth[i][j:j + 1], f"tail {i} position {j}")
        s.release([a])
    for ids in ([0, 1, 2], [3, 4, 5]):                      # unequal batches, one after the other in the same slots
        n_dec = dict(zip(ids, (3, 9, 20)))
        pos = {i: len(reqs[i]) - n_dec[i] for i in ids}
        slots = dict(zip(ids, s.begin(3)))
        got = s.step([slots[i] for i in ids], [reqs[i][:pos[i]] for i in ids])
        for k, i in enumerate(ids):
            check(got[k:k + 1], truth[i][pos[i] - 1:pos[i]], f"batch prompt {i}")
        live = list(ids)
        while live:
            got = s.step([slots[i] for i in live], [[reqs[i][pos[i]]] for i in live])
            for k, i in enumerate(live):
                check(got[k:k + 1], truth[i][pos[i]:pos[i] + 1], f"batch decode {i} at {pos[i]}")
                pos[i] += 1
            for i in [i for i in live if pos[i] == len(reqs[i])]:
                s.release([slots[i]])
                live.remove(i)
    assert s.recorded_steps() >= 2
    print(f"8B shape, bfloat16 against 32-bit: worst error {worst:.3f} of the bound")


def test_sixty_four_prompts_in_one_step(models):
    """The prompts of a batch of 64 as the generation loop issues them: in one step if they fit the
    step's token budget, else in the steps that `prefill_steps` cuts.  The last row of some of them
    against the same prompt alone; then decode steps of all 64 (tiles of 64 rows, cut along K)."""
    from picolm_amd.engine import Session
    from picolm_amd.generation import SessionStepper
    V = SHAPE["vocab_size"]
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
