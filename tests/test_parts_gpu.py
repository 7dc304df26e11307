"""Each part of a layer alone against its plain function, and a toy architecture whose mixer
keeps state of its own: defined, registered, built, loaded from a random model folder and
stepped here, without a change to the library's files."""
import json
import math
import os

import numpy as np
import pytest
import torch

import tiny
from plain import llama_plain as P

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def harness(dtype, requests, slots, pos0, new_lens, n_slots=4, max_tokens=1024):
    """A step context over a fresh cache that holds what `requests` ask for."""
    from picolm_amd.cache import Cache, CacheSpec, KVGroupSpec, StateGroupSpec
    from picolm_amd.engine.batch import StepBatch
    from picolm_amd.parts import CacheBinding, Runtime, StepContext, Workspace
    kv_req, st_req = requests
    spec = CacheSpec([KVGroupSpec(1, kv_req.n_kv_heads, kv_req.head_dim, kv_req.window, kv_req.v_head_dim)] if kv_req else [],
                     [StateGroupSpec(1, tuple(st_req.shape), st_req.dtype)] if st_req else [])
    rt = Runtime(DEV, dtype)
    cache = Cache(spec, max_tokens, 512, dtype, DEV, n_slots)
    for _ in range(n_slots):
        cache.alloc_slot()
    cache.reserve_many(slots, [p + n for p, n in zip(pos0, new_lens)])
    cache.flush()
    batch = StepBatch(slots, pos0, [[0] * n for n in new_lens], [[] for _ in slots], 10, DEV)
    ctx = StepContext(rt, batch, cache, Workspace(DEV))
    ctx.binding = CacheBinding((0, 0) if kv_req else None, (0, 0) if st_req else None, True)
    return rt, ctx


def tol(dtype, ref):
    return (3e-5 if dtype == torch.float32 else 3e-2) * max(1.0, float(np.abs(ref).max()))


def rounded(x, dtype):
    return torch.from_numpy(x).to(dtype).double().numpy()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_part(dtype):
    from picolm_amd.parts import RMSNorm
    from picolm_amd.weights import TensorDict, WeightFetcher
    rng = np.random.default_rng(0)
    w = rng.standard_normal(96)
    x = rng.standard_normal((7, 96)) * 4
    rt, ctx = harness(dtype, (None, None), [0], [0], [7])
    part = RMSNorm("n.weight", 96, 1e-3)
    assert [(s.name, s.shape, s.init) for s in part.tensor_specs()] == [("n.weight", (96,), "ones")]
    part.load_all(WeightFetcher(TensorDict({"n.weight": torch.from_numpy(w).to(torch.bfloat16)}), DEV), rt)
    out = part.forward(ctx, torch.from_numpy(x).float().to(DEV))
    ref = P.rmsnorm(x.astype(np.float32), rounded(w, torch.bfloat16), 1e-3)
    assert out.dtype == dtype and np.abs(out.double().cpu().numpy() - ref).max() <= tol(dtype, ref)
    shifted = RMSNorm("n.weight", 96, 1e-3, weight_offset=1.0)            # the convention of other architectures
    shifted.load_all(WeightFetcher(TensorDict({"n.weight": torch.from_numpy(w).float()}), DEV), rt)
    out = shifted.forward(ctx, torch.from_numpy(x).float().to(DEV))
    ref = P.rmsnorm(x.astype(np.float32), w.astype(np.float32).astype(np.float64) + 1.0, 1e-3)
    assert np.abs(out.double().cpu().numpy() - ref).max() <= tol(dtype, ref)


def test_rotary_tables():
    from picolm_amd.config import RopeScaling
    from picolm_amd.parts import RotaryEmbedding, Runtime
    sc = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=64)
    for d, theta, scaling in ((16, 10000.0, None), (32, 500000.0, sc), (128, 500000.0, dict(sc, original_max_position_embeddings=8192))):
        rot = RotaryEmbedding(d, theta, RopeScaling.from_dict(scaling), "half")
        rot.prepare(Runtime(DEV, torch.float32), 300)
        cos, sin, style = rot.rotary_tables()
        assert style == 1 and tuple(cos.shape) == (300, d // 2)
        rc, rs = P.rope_tables(np.arange(300), P.rope_inv_freq(d, theta, scaling))
        # the engine's angle is a 32-bit product: half an ulp of the largest angle
        assert np.abs(cos.double().cpu().numpy() - rc).max() < 300 * 2.0 ** -24 + 1e-7
        assert np.abs(sin.double().cpu().numpy() - rs).max() < 300 * 2.0 ** -24 + 1e-7


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,style,window", [(4, 2, 16, "pairwise", 0), (6, 6, 32, "half", 0), (8, 2, 64, "pairwise", 0),
                                                (3, 1, 32, "half", 40)])
def test_attention_part(dtype, H, G, d, style, window):
    from picolm_amd.parts import Attention, RotaryEmbedding
    from picolm_amd.weights import TensorDict, WeightFetcher
    rng = np.random.default_rng(H * d)
    D = 80
    names = ["a.q_proj.weight", "a.k_proj.weight", "a.v_proj.weight", "a.o_proj.weight"]
    shapes = [(H * d, D), (G * d, D), (G * d, D), (D, H * d)]
    w = {n: rounded(rng.standard_normal(s) * 0.2, torch.bfloat16) for n, s in zip(names, shapes)}
    part = Attention("a.", D, H, G, d, position=RotaryEmbedding(d, 1000.0, None, style), window=window)
    assert sorted(s.name for s in part.all_specs()) == sorted(names)
    lens = [70, 9] if window == 0 else [300, 9]         # longer than one chunk of a windowed group's ring
    rt, ctx = harness(dtype, part.cache_requests(), [2, 0], [0, 0], lens)
    part.load_all(WeightFetcher(TensorDict({k: torch.from_numpy(v).to(torch.bfloat16) for k, v in w.items()}), DEV), rt)
    part.prepare(rt, 512)
    hs = [rounded(rng.standard_normal((n, D)), dtype) for n in lens]
    h = torch.from_numpy(np.concatenate(hs)).to(dtype).to(DEV)
    res = torch.zeros(sum(lens), D, device=DEV)
    part.forward(ctx, h, res)
    cfg = dict(num_attention_heads=H, num_key_value_heads=G, head_dim=d, rope_theta=1000.0, rope_style=style, window=window)
    pw = {"self_attn." + k[2:]: v for k, v in w.items()}
    ref = np.concatenate([P.attention_block(x, pw, "self_attn.", cfg, np.arange(len(x))) for x in hs])
    assert np.abs(res.double().cpu().numpy() - ref).max() <= tol(dtype, ref)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_and_block_parts(dtype):
    from picolm_amd.parts import Attention, NoPosition, PreNormBlock, RMSNorm, SwiGLU
    from picolm_amd.weights import TensorDict, WeightFetcher
    rng = np.random.default_rng(5)
    D, F, H, G, d = 48, 104, 3, 3, 16
    shapes = {"f.gate_proj.weight": (F, D), "f.up_proj.weight": (F, D), "f.down_proj.weight": (D, F),
              "a.q_proj.weight": (H * d, D), "a.k_proj.weight": (G * d, D), "a.v_proj.weight": (G * d, D),
              "a.o_proj.weight": (D, H * d), "n1": (D,), "n2": (D,)}
    w = {n: rounded(rng.standard_normal(s) * 0.3, torch.bfloat16) for n, s in shapes.items()}
    ffn = SwiGLU("f.", D, F)
    block = PreNormBlock(RMSNorm("n1", D, 1e-5), Attention("a.", D, H, G, d, position=NoPosition()), RMSNorm("n2", D, 1e-5), ffn)
    rt, ctx = harness(dtype, block.mixer.cache_requests(), [1], [0], [21])
    block.load_all(WeightFetcher(TensorDict({k: torch.from_numpy(v).to(torch.bfloat16) for k, v in w.items()}), DEV), rt)
    block.mixer.prepare(rt, 512)
    x = rng.standard_normal((21, D))
    # the feed-forward alone
    hin = rounded(x, dtype)
    res = torch.zeros(21, D, device=DEV)
    ffn.forward(ctx, torch.from_numpy(hin).to(dtype).to(DEV), res)
    ref = P.swiglu(hin, w["f.gate_proj.weight"], w["f.up_proj.weight"], w["f.down_proj.weight"])
    assert np.abs(res.double().cpu().numpy() - ref).max() <= tol(dtype, ref)
    # the block: x += attn(norm(x)); x += ffn(norm(x)), here without any rotation
    xf = x.astype(np.float32).astype(np.float64)
    xt = torch.from_numpy(xf).float().to(DEV)
    block.forward(ctx, xt)
    hh = P.rmsnorm(xf, w["n1"], 1e-5)
    T = len(xf)
    q = (hh @ w["a.q_proj.weight"].T).reshape(T, H, d)
    k = (hh @ w["a.k_proj.weight"].T).reshape(T, G, d)
    v = (hh @ w["a.v_proj.weight"].T).reshape(T, G, d)
    y = xf + P.causal_attention(q, k, v).reshape(T, H * d) @ w["a.o_proj.weight"].T
    y = y + P.swiglu(P.rmsnorm(y, w["n2"], 1e-5), w["f.gate_proj.weight"], w["f.up_proj.weight"], w["f.down_proj.weight"])
    assert np.abs(xt.double().cpu().numpy() - y).max() <= tol(dtype, y)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_and_head_parts(dtype):
    from picolm_amd.parts import LMHead, TokenEmbedding
    from picolm_amd.weights import TensorDict, WeightFetcher
    rng = np.random.default_rng(6)
    V, D = 131, 40
    e, hd = rounded(rng.standard_normal((V, D)), torch.bfloat16), rounded(rng.standard_normal((V, D)), torch.bfloat16)
    rt, ctx = harness(dtype, (None, None), [0], [0], [5])
    for tied, have_head in ((True, False), (False, True), (False, False), (True, True)):
        emb = TokenEmbedding("e", V, D)
        head = LMHead("h", V, D, emb, tied)
        t = {"e": torch.from_numpy(e).to(torch.bfloat16)}
        if have_head:
            t["h"] = torch.from_numpy(hd).to(torch.bfloat16)
        f = WeightFetcher(TensorDict(t), DEV)
        emb.load_all(f, rt)
        head.load_all(f, rt)
        toks = torch.tensor([3, 130, 0, 7, 7], dtype=torch.int32, device=DEV)
        x = emb.forward(ctx, toks, 5)
        assert x.dtype == torch.float32 and np.array_equal(x.double().cpu().numpy(), e[[3, 130, 0, 7, 7]])
        hrows = rounded(rng.standard_normal((5, D)), dtype)
        lg = head.forward(ctx, torch.from_numpy(hrows).to(dtype).to(DEV))
        table = hd if (have_head and not tied) else e
        ref = hrows @ table.T
        assert np.abs(lg.double().cpu().numpy() - ref).max() <= tol(dtype, ref)


# ------------------------------------------------------------------------------------------- a toy architecture
def test_toy_architecture_with_a_stateful_mixer(tmp_path):
    """A mixer that keeps, per sequence, the running sum of its inputs and their count: its
    output at a position is W times the mean of all inputs so far.  It needs no keys or
    values, only a state row per slot.  The layer order names its block twice and the second
    call has a state entry of its own."""
    from picolm_amd.config import register_architecture, unregister_architecture
    from picolm_amd.engine import DecoderModel, Session, load_model
    from picolm_amd.parts import LMHead, Mixer, PreNormBlock, RMSNorm, StateRequest, SwiGLU, TokenEmbedding
    from picolm_amd.weights import TensorSpec, write_random_model

    class ToyConfig:
        def __init__(self, d):
            self.d = dict(d)
            self.hidden_size, self.vocab_size, self.intermediate_size = d["hidden_size"], d["vocab_size"], d["intermediate_size"]
            self.max_position_embeddings = d["max_position_embeddings"]
            self.torch_dtype = "bfloat16"
            self.eos_token_ids = ()

        def to_dict(self):
            return dict(self.d)

    class RunningMean(Mixer):
        def __init__(self, name, D):
            self.name, self.D, self.w = name, D, None

        def tensor_specs(self):
            return [TensorSpec(self.name, (self.D, self.D))]

        def load(self, fetch, runtime):
            self.w = fetch.get(self.name).float()

        def cache_requests(self):
            return None, StateRequest((self.D + 1,), torch.float32)

        def forward(self, ctx, h, residual):
            state = ctx.state()                                   # [n_slots, D + 1]
            b = ctx.batch
            row = 0
            for slot, n in zip(b.slots, b.n_new):                  # each sequence's rows in order
                x = h[row:row + n].float()
                sums = state[slot, :self.D] + torch.cumsum(x, dim=0)
                counts = state[slot, self.D] + torch.arange(1, n + 1, device=x.device, dtype=torch.float32)
                residual[row:row + n] += (sums / counts[:, None]) @ self.w.T
                state[slot, :self.D] = sums[-1]
                state[slot, self.D] = counts[-1]
                row += n

    def build(cfg):
        D = cfg.hidden_size
        emb = TokenEmbedding("emb.weight", cfg.vocab_size, D)
        block = PreNormBlock(RMSNorm("norm1.weight", D, 1e-5), RunningMean("mean.weight", D),
                             RMSNorm("norm2.weight", D, 1e-5), SwiGLU("ffn.", D, cfg.intermediate_size))
        return DecoderModel(cfg, emb, [block], RMSNorm("final.weight", D, 1e-5),
                            LMHead("head.weight", cfg.vocab_size, D, emb, tied=True), order=[0, 0])

    register_architecture("ToyRunningMeanLM", ToyConfig, build)
    try:
        cfg = ToyConfig(dict(architectures=["ToyRunningMeanLM"], hidden_size=40, vocab_size=77, intermediate_size=56,
                             max_position_embeddings=256))
        d = write_random_model(cfg, str(tmp_path / "toy"), seed=4, std=0.3)
        model = load_model(d, dtype="float32")
        assert model.cache_spec.kv_groups == [] and model.cache_spec.state_groups[0].n_entries == 2
        # the plain form of the same model
        w = tiny.read_weights_f64(d)

        def plain(tokens):
            x = w["emb.weight"][tokens]
            for _ in range(2):
                hh = P.rmsnorm(x, w["norm1.weight"], 1e-5)
                mean = np.cumsum(hh, axis=0) / np.arange(1, len(tokens) + 1)[:, None]
                x = x + mean @ w["mean.weight"].T
                x = x + P.swiglu(P.rmsnorm(x, w["norm2.weight"], 1e-5), w["ffn.gate_proj.weight"],
                                 w["ffn.up_proj.weight"], w["ffn.down_proj.weight"])
            return P.rmsnorm(x, w["final.weight"], 1e-5) @ w["emb.weight"].T
        rng = np.random.default_rng(7)
        reqs = [tiny.random_tokens(rng, n, 77) for n in (19, 3, 40)]
        truth = [plain(r) for r in reqs]
        s = Session(model, max_tokens=512, n_slots=3)
        slots = s.begin(3)                                        # whole, as one unequal batch
        got = s.step(slots, reqs, [list(range(len(r))) for r in reqs]).double().cpu().numpy()
        assert np.abs(got - np.concatenate(truth)).max() < 5e-5
        s.release(slots)
        slots = s.begin(3)                                        # reused slots: state starts from zero again
        cut = [7, 1, 33]
        s.step(slots, [r[:c] for r, c in zip(reqs, cut)])
        pos = dict(zip(range(3), cut))
        live = [0, 1, 2]
        while live:
            out = s.step([slots[i] for i in live], [[reqs[i][pos[i]]] for i in live]).double().cpu().numpy()
            for k, i in enumerate(live):
                assert np.abs(out[k] - truth[i][pos[i]]).max() < 5e-5
                pos[i] += 1
            live = [i for i in live if pos[i] < len(reqs[i])]
    finally:
        unregister_architecture("ToyRunningMeanLM")


@pytest.mark.parametrize("native", [True, False])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layer_order_names_a_block_twice_and_lets_a_call_read_anothers_cache(dtype, native, tmp_path):
    """The order of layers is data.  Three blocks of the library's own parts run as four calls:
    block 0, block 1, block 0 again (the same weights, keys and values of its own) and block 2,
    whose attention writes nothing and reads the keys and values that the call of block 1 left
    (its own k and v projections are loaded and unused).  Whole prompts as an unequal batch, then
    token by token from a cut, in the library's step and in the one from Python, against the
    plain functions."""
    from picolm_amd.config import LlamaConfig, register_architecture, unregister_architecture
    from picolm_amd.engine import DecoderModel, LayerCall, Session, load_model
    from picolm_amd.parts import Attention, LMHead, PreNormBlock, RMSNorm, RotaryEmbedding, SwiGLU, TokenEmbedding
    from picolm_amd.weights import write_random_model

    def build(cfg):
        D = cfg.hidden_size
        rotary = RotaryEmbedding(cfg.head_dim, cfg.rope_theta, cfg.rope_scaling, cfg.rope_style)
        blocks = []
        for l in range(3):
            q = f"model.layers.{l}."
            blocks.append(PreNormBlock(RMSNorm(q + "input_layernorm.weight", D, cfg.rms_norm_eps),
                                       Attention(q + "self_attn.", D, cfg.num_attention_heads, cfg.num_key_value_heads,
                                                 cfg.head_dim, position=rotary),
                                       RMSNorm(q + "post_attention_layernorm.weight", D, cfg.rms_norm_eps),
                                       SwiGLU(q + "mlp.", D, cfg.intermediate_size)))
        emb = TokenEmbedding("model.embed_tokens.weight", cfg.vocab_size, D)
        return DecoderModel(cfg, emb, blocks, RMSNorm("model.norm.weight", D, cfg.rms_norm_eps),
                            LMHead("lm_head.weight", cfg.vocab_size, D, emb, True),
                            order=[0, 1, 0, LayerCall(2, reads_cache_of=1)])

    name = "ToyOrderLM"
    register_architecture(name, LlamaConfig.from_dict, build)
    try:
        c = dict(architectures=[name], hidden_size=192, num_attention_heads=6, num_key_value_heads=2, head_dim=32,
                 intermediate_size=272, num_hidden_layers=3, vocab_size=301, rms_norm_eps=1e-5, rope_theta=10000.0,
                 max_position_embeddings=512, tie_word_embeddings=True, torch_dtype="bfloat16")
        cfg = LlamaConfig.from_dict(c)
        d = write_random_model(cfg, str(tmp_path / "order"), seed=11, std=0.06)
        model = load_model(d, dtype=dtype)
        assert [g.n_entries for g in model.cache_spec.kv_groups] == [3]      # four calls, three of them own an entry
        w = tiny.read_weights_f64(d)
        pc = dict(c, rope_style=cfg.rope_style)
        H, G, hd = 6, 2, 32

        def plain(tokens):
            T = len(tokens)
            pos = np.arange(T)
            x = w["model.embed_tokens.weight"][np.asarray(tokens)]
            kept = {}
            for call, (l, reads) in enumerate([(0, None), (1, None), (0, None), (2, 1)]):
                q_ = f"model.layers.{l}."
                h = P.rmsnorm(x, w[q_ + "input_layernorm.weight"], 1e-5)
                if reads is None:
                    x = x + P.attention_block(h, w, q_ + "self_attn.", pc, pos)
                    inv = P.rope_inv_freq(hd, 10000.0)
                    cos, sin = P.rope_tables(pos, inv)
                    kept[call] = (P.apply_rope((h @ w[q_ + "self_attn.k_proj.weight"].T).reshape(T, G, hd), cos, sin, cfg.rope_style),
                                  (h @ w[q_ + "self_attn.v_proj.weight"].T).reshape(T, G, hd))
                else:
                    inv = P.rope_inv_freq(hd, 10000.0)
                    cos, sin = P.rope_tables(pos, inv)
                    qq = P.apply_rope((h @ w[q_ + "self_attn.q_proj.weight"].T).reshape(T, H, hd), cos, sin, cfg.rope_style)
                    a = P.causal_attention(qq, kept[reads][0], kept[reads][1]).reshape(T, H * hd)
                    x = x + a @ w[q_ + "self_attn.o_proj.weight"].T
                h = P.rmsnorm(x, w[q_ + "post_attention_layernorm.weight"], 1e-5)
                x = x + P.swiglu(h, w[q_ + "mlp.gate_proj.weight"], w[q_ + "mlp.up_proj.weight"], w[q_ + "mlp.down_proj.weight"])
            return P.rmsnorm(x, w["model.norm.weight"], 1e-5) @ w["model.embed_tokens.weight"].T

        rng = np.random.default_rng(3)
        reqs = [tiny.random_tokens(rng, n, 301) for n in (150, 9, 70)]
        truth = [plain(r) for r in reqs]
        tol_ = lambda t: tiny.tolerance(dtype, t, tiny.spread(192, 0.06))
        s = Session(model, max_tokens=1024, n_slots=3, native=native)
        assert (s.engine is not None) == native
        slots = s.begin(3)
        got = s.step(slots, reqs, [list(range(len(r))) for r in reqs]).double().cpu().numpy()
        row = 0
        for r, t in zip(reqs, truth):
            assert np.abs(got[row:row + len(r)] - t).max() <= tol_(t)
            row += len(r)
        s.release(slots)
        slots = s.begin(3)                                        # the slots again, from a cut, token by token
        cut = [130, 1, 60]
        s.step(slots, [r[:c_] for r, c_ in zip(reqs, cut)])
        pos = dict(zip(range(3), cut))
        live = [0, 1, 2]
        while live:
            out = s.step([slots[i] for i in live], [[reqs[i][pos[i]]] for i in live]).double().cpu().numpy()
            for k, i in enumerate(live):
                assert np.abs(out[k] - truth[i][pos[i]]).max() <= tol_(truth[i]), (i, pos[i])
                pos[i] += 1
            live = [i for i in live if pos[i] < len(reqs[i])]
    finally:
        unregister_architecture(name)


def test_toy_mixer_whose_values_are_wider_than_its_keys(tmp_path):
    """A one-head attention defined here with keys of 16 and values of 24: the cache gives its
    group keys and values of their own sizes.  Whole prompts as an unequal batch, then the same
    requests cut into a prompt and single tokens in slots that were used before."""
    from picolm_amd.cache.slots import PAGE_TOKENS
    from picolm_amd.config import register_architecture, unregister_architecture
    from picolm_amd.engine import DecoderModel, Session, load_model
    from picolm_amd.parts import KVRequest, LMHead, Mixer, PreNormBlock, RMSNorm, SwiGLU, TokenEmbedding
    from picolm_amd.weights import TensorSpec, write_random_model
    DK, DV = 16, 24

    class ToyConfig:
        def __init__(self, d):
            self.d = dict(d)
            self.hidden_size, self.vocab_size, self.intermediate_size = d["hidden_size"], d["vocab_size"], d["intermediate_size"]
            self.max_position_embeddings = d["max_position_embeddings"]
            self.torch_dtype = "bfloat16"
            self.eos_token_ids = ()

        def to_dict(self):
            return dict(self.d)

    class NarrowKeys(Mixer):
        def __init__(self, prefix, D):
            self.prefix, self.D, self.w = prefix, D, {}

        def tensor_specs(self):
            return [TensorSpec(self.prefix + "q", (DK, self.D)), TensorSpec(self.prefix + "k", (DK, self.D)),
                    TensorSpec(self.prefix + "v", (DV, self.D)), TensorSpec(self.prefix + "o", (self.D, DV))]

        def load(self, fetch, runtime):
            self.w = {n: fetch.get(self.prefix + n).float() for n in "qkvo"}

        def cache_requests(self):
            return KVRequest(1, DK, 0, DV), None

        def forward(self, ctx, h, residual):
            k_pages, v_pages, table, _ = ctx.kv()          # [page][1][64][DK], [page][1][DV][64]
            assert k_pages.shape[-1] == DK and v_pages.shape[-2] == DV
            b, row = ctx.batch, 0
            for slot, p0, n in zip(b.slots, b.pos0, b.n_new):
                x = h[row:row + n].float()
                q, k, v = x @ self.w["q"].T, x @ self.w["k"].T, x @ self.w["v"].T
                pos = torch.arange(p0 + n, device=x.device)
                page, at = table[slot, pos // PAGE_TOKENS].long(), pos % PAGE_TOKENS
                k_pages[page[p0:], 0, at[p0:]] = k.to(k_pages.dtype)
                v_pages[page[p0:], 0, :, at[p0:]] = v.to(v_pages.dtype)
                keys, values = k_pages[page, 0, at].float(), v_pages[page, 0, :, at].float()
                s = q @ keys.T / math.sqrt(DK)
                s = s.masked_fill(pos[None, :] > pos[p0:, None], float("-inf"))
                residual[row:row + n] += (torch.softmax(s, dim=-1) @ values) @ self.w["o"].T
                row += n

    def build(cfg):
        D = cfg.hidden_size
        emb = TokenEmbedding("emb.weight", cfg.vocab_size, D)
        blocks = [PreNormBlock(RMSNorm(f"l{i}.norm1.weight", D, 1e-5), NarrowKeys(f"l{i}.mix.", D),
                               RMSNorm(f"l{i}.norm2.weight", D, 1e-5), SwiGLU(f"l{i}.ffn.", D, cfg.intermediate_size)) for i in range(2)]
        return DecoderModel(cfg, emb, blocks, RMSNorm("final.weight", D, 1e-5),
                            LMHead("head.weight", cfg.vocab_size, D, emb, tied=True))

    register_architecture("ToyNarrowKeysLM", ToyConfig, build)
    try:
        cfg = ToyConfig(dict(architectures=["ToyNarrowKeysLM"], hidden_size=40, vocab_size=77, intermediate_size=56,
                             max_position_embeddings=256))
        d = write_random_model(cfg, str(tmp_path / "toy"), seed=5, std=0.3)
        model = load_model(d, dtype="float32")
        (group,) = model.cache_spec.kv_groups
        assert (group.n_entries, group.head_dim, group.value_dim) == (2, DK, DV)
        assert model.program() is None            # a part without `emit`: stepped part by part
        w = tiny.read_weights_f64(d)

        def plain(tokens):
            x = w["emb.weight"][tokens]
            n = len(tokens)
            for i in range(2):
                hh = P.rmsnorm(x, w[f"l{i}.norm1.weight"], 1e-5)
                q, k, v = (hh @ w[f"l{i}.mix.{c}"].T for c in "qkv")
                s = q @ k.T / math.sqrt(DK)
                s[np.triu_indices(n, 1)] = -np.inf
                p = np.exp(s - s.max(axis=1, keepdims=True))
                x = x + (p / p.sum(axis=1, keepdims=True)) @ v @ w[f"l{i}.mix.o"].T
                x = x + P.swiglu(P.rmsnorm(x, w[f"l{i}.norm2.weight"], 1e-5), w[f"l{i}.ffn.gate_proj.weight"],
                                 w[f"l{i}.ffn.up_proj.weight"], w[f"l{i}.ffn.down_proj.weight"])
            return P.rmsnorm(x, w["final.weight"], 1e-5) @ w["emb.weight"].T
        rng = np.random.default_rng(8)
        reqs = [tiny.random_tokens(rng, n, 77) for n in (70, 3, 130)]
        truth = [plain(r) for r in reqs]
        s = Session(model, max_tokens=512, n_slots=3)
        assert s.cache.kv[0].k.shape[-1] == DK and s.cache.kv[0].v.shape[-2] == DV
        slots = s.begin(3)
        got = s.step(slots, reqs, [list(range(len(r))) for r in reqs]).double().cpu().numpy()
        assert np.abs(got - np.concatenate(truth)).max() < 1e-4
        s.release(slots)
        slots = s.begin(3)
        cut = [60, 1, 126]
        s.step(slots, [r[:c] for r, c in zip(reqs, cut)])
        pos, live = dict(zip(range(3), cut)), [0, 1, 2]
        while live:
            out = s.step([slots[i] for i in live], [[reqs[i][pos[i]]] for i in live]).double().cpu().numpy()
            for k, i in enumerate(live):
                assert np.abs(out[k] - truth[i][pos[i]]).max() < 1e-4
                pos[i] += 1
            live = [i for i in live if pos[i] < len(reqs[i])]
    finally:
        unregister_architecture("ToyNarrowKeysLM")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_toy_position_encoding_that_is_no_rotation(dtype):
    """A position encoding defined here: it damps queries and keys with their position.  The
    attention part takes it through `PositionEncoding.apply`, in a prefill step and in decode steps
    (where the bfloat16 kernel that writes the cache itself gets rows that are already encoded)."""
    from picolm_amd.cache.slots import PAGE_TOKENS
    from picolm_amd.engine.batch import StepBatch
    from picolm_amd.parts import Attention, PositionEncoding
    from picolm_amd.weights import TensorDict, WeightFetcher

    class Damping(PositionEncoding):
        """q and k of the token at position p are multiplied by 1 / (1 + p / 32)."""

        def apply(self, ctx, qkv, H, G, d):
            f = 1.0 / (1.0 + ctx.batch.tok_pos[:qkv.shape[0]].float() / 32.0)
            qkv[:, :(H + G) * d] *= f[:, None]

    H, G, d, D = 4, 2, 32, 48
    rng = np.random.default_rng(9)
    names = ["a.q_proj.weight", "a.k_proj.weight", "a.v_proj.weight", "a.o_proj.weight"]
    shapes = [(H * d, D), (G * d, D), (G * d, D), (D, H * d)]
    w = {n: rounded(rng.standard_normal(s) * 0.2, torch.bfloat16) for n, s in zip(names, shapes)}
    part = Attention("a.", D, H, G, d, position=Damping())
    lens, tail = [70, 9], 3
    rt, ctx = harness(dtype, part.cache_requests(), [2, 0], [0, 0], [n + tail for n in lens])
    part.load_all(WeightFetcher(TensorDict({k: torch.from_numpy(v).to(torch.bfloat16) for k, v in w.items()}), DEV), rt)
    part.prepare(rt, 512)
    hs = [rounded(rng.standard_normal((n + tail, D)), dtype) for n in lens]

    def plain(x):
        T = len(x)
        f = 1.0 / (1.0 + np.arange(T) / 32.0)
        q = (x @ w["a.q_proj.weight"].T).reshape(T, H, d) * f[:, None, None]
        k = (x @ w["a.k_proj.weight"].T).reshape(T, G, d) * f[:, None, None]
        v = (x @ w["a.v_proj.weight"].T).reshape(T, G, d)
        return P.causal_attention(q, k, v).reshape(T, H * d) @ w["a.o_proj.weight"].T
    ref = [plain(x) for x in hs]
    # the prompts in one step, then one token each
    ctx.batch = StepBatch([2, 0], [0, 0], [[0] * n for n in lens], [[], []], 10, DEV)
    res = torch.zeros(sum(lens), D, device=DEV)
    part.forward(ctx, torch.from_numpy(np.concatenate([x[:n] for x, n in zip(hs, lens)])).to(dtype).to(DEV), res)
    want = np.concatenate([r[:n] for r, n in zip(ref, lens)])
    assert np.abs(res.double().cpu().numpy() - want).max() <= tol(dtype, want)
    for j in range(tail):
        ctx.batch = StepBatch([2, 0], [n + j for n in lens], [[0], [0]], [[], []], 10, DEV)
        res = torch.zeros(2, D, device=DEV)
        part.forward(ctx, torch.from_numpy(np.stack([x[n + j] for x, n in zip(hs, lens)])).to(dtype).to(DEV), res)
        want = np.stack([r[n + j] for r, n in zip(ref, lens)])
        assert np.abs(res.double().cpu().numpy() - want).max() <= tol(dtype, want)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_norm_that_is_no_rmsnorm(dtype, tmp_path):
    """A norm of another kind, defined here: it subtracts the row's mean, divides by the standard
    deviation and has a weight and a bias.  The products around a norm share an RMSNorm between
    them in decode steps; this one says nothing of the kind (`rms_parameters` is None), so its
    own `forward` must run wherever it stands: before the mixer, before the feed-forward, and as
    the last norm of one block with an RMSNorm following in the next.  Prompts whole, then token by
    token (where the sharing would happen), against the plain functions."""
    from picolm_amd.config import LlamaConfig, register_architecture, unregister_architecture
    from picolm_amd.engine import DecoderModel, Session, load_model
    from picolm_amd.parts import Attention, LMHead, Norm, PreNormBlock, RMSNorm, RotaryEmbedding, SwiGLU, TokenEmbedding
    from picolm_amd.weights import TensorSpec, write_random_model

    class CenteredNorm(Norm):
        def __init__(self, name, size, eps):
            self.name, self.size, self.eps = name, size, eps
            self.weight = self.bias = None

        def tensor_specs(self):
            return [TensorSpec(self.name + ".weight", (self.size,), init="ones"), TensorSpec(self.name + ".bias", (self.size,))]

        def load(self, fetch, runtime):
            self.weight = fetch.get(self.name + ".weight").float()
            self.bias = fetch.get(self.name + ".bias").float()

        def forward(self, ctx, x, rows=None, n_rows=None, out_name="norm.out"):
            if rows is not None:
                x = x[rows[:n_rows].long()] if n_rows is not None else x[rows.long()]
            xc = x - x.mean(dim=1, keepdim=True)
            y = xc * torch.rsqrt((xc * xc).mean(dim=1, keepdim=True) + self.eps) * self.weight + self.bias
            return y.to(ctx.dtype)

    def build(cfg):
        D = cfg.hidden_size
        rotary = RotaryEmbedding(cfg.head_dim, cfg.rope_theta, cfg.rope_scaling, cfg.rope_style)
        blocks = []
        for l in range(2):
            q = f"model.layers.{l}."
            first = CenteredNorm(q + "input_norm", D, 1e-5) if l == 0 else RMSNorm(q + "input_layernorm.weight", D, 1e-5)
            second = RMSNorm(q + "post_attention_layernorm.weight", D, 1e-5) if l == 0 else CenteredNorm(q + "post_norm", D, 1e-5)
            blocks.append(PreNormBlock(first, Attention(q + "self_attn.", D, cfg.num_attention_heads, cfg.num_key_value_heads,
                                                        cfg.head_dim, position=rotary),
                                       second, SwiGLU(q + "mlp.", D, cfg.intermediate_size)))
        emb = TokenEmbedding("model.embed_tokens.weight", cfg.vocab_size, D)
        return DecoderModel(cfg, emb, blocks, CenteredNorm("model.final_norm", D, 1e-5),
                            LMHead("lm_head.weight", cfg.vocab_size, D, emb, True))

    name = "ToyCenteredNormLM"
    register_architecture(name, LlamaConfig.from_dict, build)
    try:
        c = dict(architectures=[name], hidden_size=128, num_attention_heads=4, num_key_value_heads=2, head_dim=32,
                 intermediate_size=192, num_hidden_layers=2, vocab_size=211, rms_norm_eps=1e-5, rope_theta=10000.0,
                 max_position_embeddings=256, tie_word_embeddings=True, torch_dtype="bfloat16")
        cfg = LlamaConfig.from_dict(c)
        d = write_random_model(cfg, str(tmp_path / "centered"), seed=5, std=0.08)
        model = load_model(d, dtype=dtype)
        w = tiny.read_weights_f64(d)
        pc = dict(c, rope_style=cfg.rope_style)

        def centered(x, n):
            xc = x - x.mean(axis=1, keepdims=True)
            return xc / np.sqrt((xc * xc).mean(axis=1, keepdims=True) + 1e-5) * w[n + ".weight"] + w[n + ".bias"]

        def plain(tokens):
            pos = np.arange(len(tokens))
            x = w["model.embed_tokens.weight"][np.asarray(tokens)]
            x = x + P.attention_block(centered(x, "model.layers.0.input_norm"), w, "model.layers.0.self_attn.", pc, pos)
            h = P.rmsnorm(x, w["model.layers.0.post_attention_layernorm.weight"], 1e-5)
            x = x + P.swiglu(h, w["model.layers.0.mlp.gate_proj.weight"], w["model.layers.0.mlp.up_proj.weight"], w["model.layers.0.mlp.down_proj.weight"])
            h = P.rmsnorm(x, w["model.layers.1.input_layernorm.weight"], 1e-5)
            x = x + P.attention_block(h, w, "model.layers.1.self_attn.", pc, pos)
            h = centered(x, "model.layers.1.post_norm")
            x = x + P.swiglu(h, w["model.layers.1.mlp.gate_proj.weight"], w["model.layers.1.mlp.up_proj.weight"], w["model.layers.1.mlp.down_proj.weight"])
            return centered(x, "model.final_norm") @ w["model.embed_tokens.weight"].T

        rng = np.random.default_rng(9)
        reqs = [tiny.random_tokens(rng, n, 211) for n in (70, 5, 33)]
        truth = [plain(r) for r in reqs]
        tol_ = lambda t: tiny.tolerance(dtype, t, tiny.spread(128, 0.08))
        s = Session(model, max_tokens=512, n_slots=3)
        assert s.engine is None                       # a part the library has no operations for: stepped from Python
        slots = s.begin(3)
        got = s.step(slots, reqs, [list(range(len(r))) for r in reqs]).double().cpu().numpy()
        row = 0
        for r, t in zip(reqs, truth):
            assert np.abs(got[row:row + len(r)] - t).max() <= tol_(t)
            row += len(r)
        s.release(slots)
        slots = s.begin(3)
        cut = [50, 2, 20]
        s.step(slots, [r[:c_] for r, c_ in zip(reqs, cut)])
        pos = dict(zip(range(3), cut))
        live = [0, 1, 2]
        while live:
            out = s.step([slots[i] for i in live], [[reqs[i][pos[i]]] for i in live]).double().cpu().numpy()
            for k, i in enumerate(live):
                assert np.abs(out[k] - truth[i][pos[i]]).max() <= tol_(truth[i]), (i, pos[i])
                pos[i] += 1
            live = [i for i in live if pos[i] < len(reqs[i])]
    finally:
        unregister_architecture(name)


def test_toy_feed_forward_with_routing():
    """A feed-forward defined here: two gated experts and a router that sends every row to the
    expert with the larger logit (router logits in float).  It is built from the library's Linear
    and SwiGLU parts and runs in a block next to attention, without a change to the library."""
    from picolm_amd.parts import FeedForward, Linear, SwiGLU
    from picolm_amd.weights import TensorDict, WeightFetcher

    class TwoExperts(FeedForward):
        def __init__(self, prefix, D, F):
            self.router = Linear([prefix + "router.weight"], [2], D)
            self.experts = [SwiGLU(prefix + f"experts.{i}.", D, F) for i in range(2)]

        def children(self):
            return [self.router] + self.experts

        def forward(self, ctx, h, residual):
            logits = torch.zeros(h.shape[0], 2, device=h.device)
            self.router.forward(h, logits)
            choice = logits.argmax(dim=1)
            for i, expert in enumerate(self.experts):
                rows = torch.nonzero(choice == i).flatten()
                if rows.numel():
                    out = torch.zeros(rows.numel(), residual.shape[1], device=h.device)
                    expert.forward(ctx, h.index_select(0, rows).contiguous(), out)
                    residual.index_add_(0, rows, out)

    D, F, T = 64, 96, 37
    rng = np.random.default_rng(3)
    shapes = {"f.router.weight": (2, D)}
    for i in range(2):
        shapes.update({f"f.experts.{i}.gate_proj.weight": (F, D), f"f.experts.{i}.up_proj.weight": (F, D),
                       f"f.experts.{i}.down_proj.weight": (D, F)})
    w = {n: rounded(rng.standard_normal(s) * 0.3, torch.bfloat16) for n, s in shapes.items()}
    ffn = TwoExperts("f.", D, F)
    assert sorted(s.name for s in ffn.all_specs()) == sorted(shapes)
    rt, ctx = harness(torch.bfloat16, (None, None), [0], [0], [T])
    ffn.load_all(WeightFetcher(TensorDict({k: torch.from_numpy(v).to(torch.bfloat16) for k, v in w.items()}), DEV), rt)
    x = rounded(rng.standard_normal((T, D)), torch.bfloat16)
    res = torch.zeros(T, D, device=DEV)
    ffn.forward(ctx, torch.from_numpy(x).to(torch.bfloat16).to(DEV), res)
    choice = (x @ w["f.router.weight"].T).argmax(axis=1)
    assert 0 < choice.sum() < T                          # both experts get rows
    ref = np.stack([P.swiglu(x[t:t + 1], w[f"f.experts.{c}.gate_proj.weight"], w[f"f.experts.{c}.up_proj.weight"],
                             w[f"f.experts.{c}.down_proj.weight"])[0] for t, c in enumerate(choice)])
    assert np.abs(res.double().cpu().numpy() - ref).max() <= tol(torch.bfloat16, ref)


# ------------------------------------------------------------------------------------------- a window's ring, lap after lap
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [40, 100])
def test_a_window_of_keys_through_several_laps_of_its_ring(dtype, window, tmp_path):
    """A decoder whose attention keeps a window of keys: its cache group is a ring of pages per
    slot.  A prompt longer than one chunk, then decoding far past the ring's first lap, launched
    step by step and replayed from the recording; every step against the plain implementation
    with the same window.  (Such a model is stepped from Python: the engine keeps all keys.)"""
    from picolm_amd import LlamaConfig
    from picolm_amd.engine import DecoderModel, Session
    from picolm_amd.parts import (Attention, LMHead, PreNormBlock, RMSNorm, RotaryEmbedding, Runtime, SwiGLU, TokenEmbedding)
    from picolm_amd.weights import Checkpoint, write_random_model
    cfgd = dict(tiny.TINY_C, max_position_embeddings=1024, num_hidden_layers=2)
    cfg = LlamaConfig.from_dict(cfgd)
    d = write_random_model(cfg, str(tmp_path / "m"), seed=6, std=0.08, norm_sigma=0.1)
    D = cfg.hidden_size
    rotary = RotaryEmbedding(cfg.head_dim, cfg.rope_theta, None, cfg.rope_style)
    blocks = [PreNormBlock(RMSNorm(f"model.layers.{l}.input_layernorm.weight", D, cfg.rms_norm_eps),
                           Attention(f"model.layers.{l}.self_attn.", D, cfg.num_attention_heads, cfg.num_key_value_heads,
                                     cfg.head_dim, position=rotary, window=window),
                           RMSNorm(f"model.layers.{l}.post_attention_layernorm.weight", D, cfg.rms_norm_eps),
                           SwiGLU(f"model.layers.{l}.mlp.", D, cfg.intermediate_size)) for l in range(2)]
    emb = TokenEmbedding("model.embed_tokens.weight", cfg.vocab_size, D)
    model = DecoderModel(cfg, emb, blocks, RMSNorm("model.norm.weight", D, cfg.rms_norm_eps),
                         LMHead("lm_head.weight", cfg.vocab_size, D, emb, False))
    ck = Checkpoint(d)
    model.load(ck, Runtime(DEV, dtype))
    ck.close()
    rng = np.random.default_rng(window)
    n_prompt, n_all = 300, 640
    toks = tiny.random_tokens(rng, n_all, cfg.vocab_size)
    ref = P.forward(tiny.read_weights_f64(d), dict(tiny.read_config(d), window=window), toks)
    for graphs in (False, True):
        s = Session(model, max_tokens=2048, graphs=graphs)
        assert s.engine is None                                   # a window is stepped from Python
        ring = s.cache.kv[0].ring_pages
        assert ring < s.cache.max_pages and 64 * ring < n_all - 64      # decoding laps the ring more than once
        [a] = s.begin(1)
        got = s.step([a], [toks[:n_prompt]], [list(range(n_prompt))]).double().cpu().numpy()
        assert np.abs(got - ref[:n_prompt]).max() <= tol(dtype, ref)
        for j in range(n_prompt, n_all):
            got = s.step([a], [[toks[j]]]).double().cpu().numpy()
            err = np.abs(got[0] - ref[j]).max()
            assert err <= tol(dtype, ref), (window, dtype, "graphs", graphs, "position", j, err)
        assert (s.recorded_steps() > 0) == graphs
        assert len(s.cache.kv[0].book.pages[a]) == ring           # the slot never holds more than its ring
        s.release([a])


@pytest.mark.parametrize("window", [40, 60])
def test_the_edge_of_a_window_in_decode_steps_past_the_first_lap(window):
    """One head whose query, key and value are the input row itself.  Two rows stand out: their
    keys score far above all others for every later query, so a decode step's output is that
    row's value while the row is inside the window and small once it has left.  The last step
    that sees it has it exactly at position - window + 1; the next one must drop it, also when its
    page of the ring has meanwhile been written again."""
    from picolm_amd.engine.batch import StepBatch
    from picolm_amd.parts import Attention
    from picolm_amd.weights import TensorDict, WeightFetcher
    d = 16
    eye = torch.eye(d)
    part = Attention("a.", d, 1, 1, d, window=window)
    from picolm_amd.cache.kv import window_ring_pages
    ring = window_ring_pages(window)
    n_prompt, n_all = 300, 64 * ring + 5 + window + 8          # (the harness's cache takes sequences of 512)
    rt, ctx = harness(torch.float32, part.cache_requests(), [1], [0], [n_all], max_tokens=1024)
    assert ctx.cache.kv[0].ring_pages == ring and n_all <= 512
    part.load_all(WeightFetcher(TensorDict({f"a.{n}_proj.weight": eye.clone() for n in "qkvo"}), DEV), rt)
    rng = np.random.default_rng(window)
    u = np.zeros(d)
    u[3] = 1.0
    h = rng.standard_normal((n_all, d)) * 0.05
    h[:, 3] = 1.0                                  # every query looks along u
    big = [305, 64 * ring + 5]                     # one in the first lap, one just after the ring has wrapped; never both in a window
    for j in big:
        h[j] = 60.0 * u                            # score 60 / 4 = 15 against about 0.25 for the others
    ref = P.causal_attention(h[:, None, :], h[:, None, :], h[:, None, :], window)[:, 0, :]
    ctx.batch = StepBatch([1], [0], [[0] * n_prompt], [[]], 10, DEV)
    res = torch.zeros(n_prompt, d, device=DEV)
    part.forward(ctx, torch.from_numpy(h[:n_prompt]).float().to(DEV), res)
    assert np.abs(res.double().cpu().numpy() - ref[:n_prompt]).max() <= 1e-4
    for p in range(n_prompt, n_all):
        ctx.batch = StepBatch([1], [p], [[0]], [[]], 10, DEV)
        res = torch.zeros(1, d, device=DEV)
        part.forward(ctx, torch.from_numpy(h[p:p + 1]).float().to(DEV), res)
        out = res.double().cpu().numpy()[0]
        assert np.abs(out - ref[p]).max() <= 1e-4, p
        for j in big:
            if p == j + window - 1:
                assert out[3] > 50.0, (p, "the key at position - window + 1 is visible")
            if p == j + window:
                assert out[3] < 2.0, (p, "the key at position - window is dropped")
