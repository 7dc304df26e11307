"""Each part of a layer alone against its plain function, and toy architectures whose parts are
defined here: registered, built, loaded from a random model folder and stepped by the engine,
without a change to the library's files.  A part written in Python (its `forward` runs torch
operators on the engine's memory) and a part with HIP kernels of its own (tests/toy_parts) both run
inside the library's step, through its cache, its planner and its generation loop."""
import ctypes
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


def tol(dtype, ref):
    return (3e-5 if dtype == torch.float32 else 3e-2) * max(1.0, float(np.abs(ref).max()))


def rounded(x, dtype):
    return torch.from_numpy(x).to(dtype).double().numpy()


def fetcher(tensors, dtype=torch.bfloat16):
    from picolm_amd.weights import TensorDict, WeightFetcher
    return WeightFetcher(TensorDict({k: torch.from_numpy(np.ascontiguousarray(v)).to(dtype) for k, v in tensors.items()}), DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_part(dtype):
    from part_harness import PartEngine
    from picolm_amd.engine import program as Pr
    from picolm_amd.parts import RMSNorm, Runtime
    rng = np.random.default_rng(0)
    w = rng.standard_normal(96)
    x = (rng.standard_normal((7, 96)) * 4).astype(np.float32)
    rt = Runtime(DEV, dtype)
    part = RMSNorm("n.weight", 96, 1e-3)
    assert [(s.name, s.shape, s.init) for s in part.tensor_specs()] == [("n.weight", (96,), "ones")]
    part.load_all(fetcher({"n.weight": w}), rt)
    shifted = RMSNorm("n.weight", 96, 1e-3, weight_offset=1.0)            # the convention of other architectures
    shifted.load_all(fetcher({"n.weight": w}, torch.float32), rt)
    for norm, weights in ((part, rounded(w, torch.bfloat16)), (shifted, w.astype(np.float32).astype(np.float64) + 1.0)):
        # as a part's input it is a norm that a product may carry; alone it runs as an operation of its own
        def emit(b, xb, h, norm=norm):
            src = norm.emit(b, xb)
            assert src.norm is not None and src.x == xb
            return b.materialize(src), 96
        e = PartEngine(dtype, x, emit, parts=[norm])
        out = e.step(e.alloc(1), [range(7)])
        ref = P.rmsnorm(x, weights, 1e-3)
        assert np.abs(out - ref).max() <= tol(dtype, ref)
    # on the wanted rows only, as before the head
    e = PartEngine(dtype, x, lambda b, xb, h: (b.materialize(part.emit(b, xb, Pr.ROWS_WANTED), Pr.ROWS_WANTED), 96), parts=[part],
                   read_rows=Pr.ROWS_WANTED)
    out = e.step(e.alloc(1), [range(7)], [[5, 0, 5]])
    ref = P.rmsnorm(x, rounded(w, torch.bfloat16), 1e-3)[[5, 0, 5]]
    assert np.abs(out - ref).max() <= tol(dtype, ref)


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


def attention_engine(dtype, part, rows, **kw):
    """The attention part alone: input rows in the compute dtype, its output added to zeros."""
    from part_harness import PartEngine
    from picolm_amd.engine.program import Rows
    D = rows.shape[1]

    def emit(b, x, h):
        res = h.zeros(b, part.o.out_size)
        part.emit(b, Rows(h.cast(b, x, D)), res)
        return res, part.o.out_size
    return PartEngine(dtype, rows, emit, requests=part.cache_requests(), parts=[part], **kw)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,style,window", [(4, 2, 16, "pairwise", 0), (6, 6, 32, "half", 0), (8, 2, 64, "pairwise", 0),
                                                (3, 1, 32, "half", 40)])
def test_attention_part(dtype, H, G, d, style, window):
    from picolm_amd.parts import Attention, RotaryEmbedding, Runtime
    rng = np.random.default_rng(H * d)
    D = 80
    names = ["a.q_proj.weight", "a.k_proj.weight", "a.v_proj.weight", "a.o_proj.weight"]
    shapes = [(H * d, D), (G * d, D), (G * d, D), (D, H * d)]
    w = {n: rounded(rng.standard_normal(s) * 0.2, torch.bfloat16) for n, s in zip(names, shapes)}
    part = Attention("a.", D, H, G, d, position=RotaryEmbedding(d, 1000.0, None, style), window=window)
    assert sorted(s.name for s in part.all_specs()) == sorted(names)
    lens = [70, 9] if window == 0 else [300, 9]         # longer than one chunk of a windowed group's ring
    part.load_all(fetcher(w), Runtime(DEV, dtype))
    hs = [rounded(rng.standard_normal((n, D)), dtype) for n in lens]
    e = attention_engine(dtype, part, np.concatenate(hs))
    slots = e.alloc(3)
    got = e.step([slots[2], slots[0]], [range(lens[0]), range(lens[0], sum(lens))])
    cfg = dict(num_attention_heads=H, num_key_value_heads=G, head_dim=d, rope_theta=1000.0, rope_style=style, window=window)
    pw = {"self_attn." + k[2:]: v for k, v in w.items()}
    ref = np.concatenate([P.attention_block(x, pw, "self_attn.", cfg, np.arange(len(x))) for x in hs])
    assert np.abs(got - ref).max() <= tol(dtype, ref)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_and_block_parts(dtype):
    from part_harness import PartEngine
    from picolm_amd.engine.program import Rows
    from picolm_amd.parts import Attention, NoPosition, PreNormBlock, RMSNorm, Runtime, SwiGLU
    rng = np.random.default_rng(5)
    D, F, H, G, d = 48, 104, 3, 3, 16
    shapes = {"f.gate_proj.weight": (F, D), "f.up_proj.weight": (F, D), "f.down_proj.weight": (D, F),
              "a.q_proj.weight": (H * d, D), "a.k_proj.weight": (G * d, D), "a.v_proj.weight": (G * d, D),
              "a.o_proj.weight": (D, H * d), "n1": (D,), "n2": (D,)}
    w = {n: rounded(rng.standard_normal(s) * 0.3, torch.bfloat16) for n, s in shapes.items()}
    ffn = SwiGLU("f.", D, F)
    block = PreNormBlock(RMSNorm("n1", D, 1e-5), Attention("a.", D, H, G, d, position=NoPosition()), RMSNorm("n2", D, 1e-5), ffn)
    block.load_all(fetcher(w), Runtime(DEV, dtype))
    x = rng.standard_normal((21, D))
    # the feed-forward alone
    hin = rounded(x, dtype)

    def emit_ffn(b, xb, h):
        res = h.zeros(b, D)
        ffn.emit(b, Rows(h.cast(b, xb, D)), res)
        return res, D
    e = PartEngine(dtype, hin, emit_ffn, parts=[ffn])
    got = e.step(e.alloc(1), [range(21)])
    ref = P.swiglu(hin, w["f.gate_proj.weight"], w["f.up_proj.weight"], w["f.down_proj.weight"])
    assert np.abs(got - ref).max() <= tol(dtype, ref)
    # the block: x += attn(norm(x)); x += ffn(norm(x)), here without any rotation
    xf = x.astype(np.float32).astype(np.float64)

    def emit_block(b, xb, h):
        block.emit(b, xb)
        return xb, D
    e = PartEngine(dtype, xf, emit_block, requests=block.mixer.cache_requests(), parts=[block, block.mixer])
    got = e.step([e.alloc(2)[1]], [range(21)])
    hh = P.rmsnorm(xf, w["n1"], 1e-5)
    T = len(xf)
    q = (hh @ w["a.q_proj.weight"].T).reshape(T, H, d)
    k = (hh @ w["a.k_proj.weight"].T).reshape(T, G, d)
    v = (hh @ w["a.v_proj.weight"].T).reshape(T, G, d)
    y = xf + P.causal_attention(q, k, v).reshape(T, H * d) @ w["a.o_proj.weight"].T
    y = y + P.swiglu(P.rmsnorm(y, w["n2"], 1e-5), w["f.gate_proj.weight"], w["f.up_proj.weight"], w["f.down_proj.weight"])
    assert np.abs(got - y).max() <= tol(dtype, y)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_and_head_parts(dtype):
    from part_harness import PartEngine
    from picolm_amd.engine import program as Pr
    from picolm_amd.engine.native import NativeEngine
    from picolm_amd.cache import CacheSpec
    from picolm_amd.parts import LMHead, Runtime, TokenEmbedding
    rng = np.random.default_rng(6)
    V, D = 131, 40
    e_, hd = rounded(rng.standard_normal((V, D)), torch.bfloat16), rounded(rng.standard_normal((V, D)), torch.bfloat16)
    rt = Runtime(DEV, dtype)
    hrows = rounded(rng.standard_normal((5, D)), dtype)
    for tied, have_head in ((True, False), (False, True), (False, False), (True, True)):
        emb = TokenEmbedding("e", V, D)
        head = LMHead("h", V, D, emb, tied)
        t = {"e": e_}
        if have_head:
            t["h"] = hd
        f = fetcher(t)
        emb.load_all(f, rt)
        head.load_all(f, rt)
        # the embedding: a program of its lookup and a read-out of the residual rows as "logits"
        b = Pr.ProgramBuilder(dtype)
        x = emb.emit(b)
        lg = b.buffer("logits", V, torch.float32, Pr.ROWS_WANTED)

        def read(view):
            from picolm_amd.parts.base import rows_view
            src = rows_view(view.inp, view.n_tokens, view.in_row_bytes, torch.float32, DEV)
            rows_view(view.out, view.n_wanted, view.out_row_bytes, torch.float32, DEV)[:, :D] = src
        b.call(read, out=lg, inp=x, rows=Pr.ROWS_WANTED)
        b.logits_buffer = lg
        eng = NativeEngine(b.finish(V, CacheSpec([], [])), 64, 64, 1, DEV)
        got = eng.step([eng.slot_alloc()], [[3, 130, 0, 7, 7]], [list(range(5))])[:, :D]
        assert got.dtype == torch.float32 and np.array_equal(got.double().cpu().numpy(), e_[[3, 130, 0, 7, 7]])
        # the head: wanted rows in the compute dtype in, logits out
        pe = PartEngine(dtype, hrows, lambda b, xb, h: (head.emit(b, h.cast(b, xb, D, Pr.ROWS_WANTED, "norm.final")) or "logits", V),
                        parts=[head])
        got = pe.step(pe.alloc(1), [range(5)])
        table = hd if (have_head and not tied) else e_
        ref = hrows @ table.T
        assert np.abs(got[:, :V] - ref).max() <= tol(dtype, ref)


# ------------------------------------------------------------------------------------------- a toy architecture
def test_toy_architecture_with_a_stateful_mixer(tmp_path):
    """A mixer that keeps, per sequence, the running sum of its inputs and their count: its
    output at a position is W times the mean of all inputs so far.  It needs no keys or
    values, only a state row per slot.  The layer order names its block twice and the second
    call has a state entry of its own."""
    from picolm_amd import SamplingParams
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
        assert tuple(s.cache.state[0].shape) == (2, 3, 41)         # the engine holds the state: [entry][slot][D + 1]
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
        assert s.recorded_steps() == 0                            # a part that runs torch operators: its steps are launched
        s.release(slots)
        # the library's generation loop steps it too: greedy tokens against the plain implementation
        toks, _ = s.engine.generate([r[:5] for r in reqs], 6, SamplingParams(), [], batch_size=2)
        for r, got in zip(reqs, toks):
            seq = list(r[:5])
            for t in got:
                row = plain(np.asarray(seq))[-1]
                assert row[t] >= row.max() - 1e-4
                seq.append(t)
    finally:
        unregister_architecture("ToyRunningMeanLM")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layer_order_names_a_block_twice_and_lets_a_call_read_anothers_cache(dtype, tmp_path):
    """The order of layers is data.  Three blocks of the library's own parts run as four calls:
    block 0, block 1, block 0 again (the same weights, keys and values of its own) and block 2,
    whose attention writes nothing and reads the keys and values that the call of block 1 left
    (its own k and v projections are loaded and unused).  Whole prompts as an unequal batch, then
    token by token from a cut, against the plain functions."""
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
        s = Session(model, max_tokens=1024, n_slots=3)
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
    from picolm_amd.cache import PAGE_TOKENS
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
            k_pages, v_pages, table, _ = ctx.kv()          # [page][1][64][DK], [page][1][DV][64]: the engine's memory
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
    attention part emits it as a call of its `apply` on the float rows of q, k, v, between the
    product and the attention operation, in a prefill step and in decode steps (where the
    bfloat16 kernel that writes the cache itself gets rows that are already encoded)."""
    from picolm_amd.parts import Attention, PositionEncoding, Runtime

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
    part.load_all(fetcher(w), Runtime(DEV, dtype))
    hs = [rounded(rng.standard_normal((n + tail, D)), dtype) for n in lens]
    first = [0, lens[0] + tail]                         # where each sequence's rows start in the table

    def plain(x):
        T = len(x)
        f = 1.0 / (1.0 + np.arange(T) / 32.0)
        q = (x @ w["a.q_proj.weight"].T).reshape(T, H, d) * f[:, None, None]
        k = (x @ w["a.k_proj.weight"].T).reshape(T, G, d) * f[:, None, None]
        v = (x @ w["a.v_proj.weight"].T).reshape(T, G, d)
        return P.causal_attention(q, k, v).reshape(T, H * d) @ w["a.o_proj.weight"].T
    ref = [plain(x) for x in hs]
    e = attention_engine(dtype, part, np.concatenate(hs))
    assert sum(op.kind == 5 for op in e.builder.ops) == 4          # the cast, the zeros, the encoding and the read-out are calls
    slots = e.alloc(3)
    slots = [slots[2], slots[0]]
    # the prompts in one step, then one token each
    got = e.step(slots, [range(f, f + n) for f, n in zip(first, lens)])
    want = np.concatenate([r[:n] for r, n in zip(ref, lens)])
    assert np.abs(got - want).max() <= tol(dtype, want)
    for j in range(tail):
        got = e.step(slots, [[f + n + j] for f, n in zip(first, lens)])
        want = np.stack([r[n + j] for r, n in zip(ref, lens)])
        assert np.abs(got - want).max() <= tol(dtype, want)


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
    and SwiGLU parts, whose `forward` it calls on the rows it picks, and runs inside the engine's
    step as a call of its own `forward`, without a change to the library."""
    from part_harness import PartEngine
    from picolm_amd.engine.program import Rows
    from picolm_amd.parts import FeedForward, Linear, Runtime, SwiGLU

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
    ffn.load_all(fetcher(w), Runtime(DEV, torch.bfloat16))
    x = rounded(rng.standard_normal((T, D)), torch.bfloat16)

    def emit(b, xb, h):
        res = h.zeros(b, D)
        ffn.emit(b, Rows(h.cast(b, xb, D)), res)
        return res, D
    e = PartEngine(torch.bfloat16, x, emit, parts=[ffn])
    got = e.step(e.alloc(1), [range(T)])
    choice = (x @ w["f.router.weight"].T).argmax(axis=1)
    assert 0 < choice.sum() < T                          # both experts get rows
    ref = np.stack([P.swiglu(x[t:t + 1], w[f"f.experts.{c}.gate_proj.weight"], w[f"f.experts.{c}.up_proj.weight"],
                             w[f"f.experts.{c}.down_proj.weight"])[0] for t, c in enumerate(choice)])
    assert np.abs(got - ref).max() <= tol(torch.bfloat16, ref)


# ------------------------------------------------------------------------------------------- a window's ring, lap after lap
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [40, 100])
def test_a_window_of_keys_through_several_laps_of_its_ring(dtype, window, tmp_path):
    """A decoder whose attention keeps a window of keys: its cache group is a ring of pages per
    slot.  A prompt longer than one chunk, then decoding far past the ring's first lap, launched
    step by step and replayed from the recording; every step against the plain implementation
    with the same window."""
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
        assert len(s.engine.slot_pages(0, a)) == ring             # the slot never holds more than its ring
        s.release([a])


@pytest.mark.parametrize("window", [40, 60])
def test_the_edge_of_a_window_in_decode_steps_past_the_first_lap(window):
    """One head whose query, key and value are the input row itself.  Two rows stand out: their
    keys score far above all others for every later query, so a decode step's output is that
    row's value while the row is inside the window and small once it has left.  The last step
    that sees it has it exactly at position - window + 1; the next one must drop it, also when its
    page of the ring has meanwhile been written again."""
    from picolm_amd.cache import window_ring_pages
    from picolm_amd.parts import Attention, Runtime
    d = 16
    eye = np.eye(d)
    part = Attention("a.", d, 1, 1, d, window=window)
    ring = window_ring_pages(window)
    n_prompt, n_all = 300, 64 * ring + 5 + window + 8          # (the cache takes sequences of 512)
    assert n_all <= 512
    part.load_all(fetcher({f"a.{n}_proj.weight": eye for n in "qkvo"}), Runtime(DEV, torch.float32))
    rng = np.random.default_rng(window)
    u = np.zeros(d)
    u[3] = 1.0
    h = rng.standard_normal((n_all, d)) * 0.05
    h[:, 3] = 1.0                                  # every query looks along u
    big = [305, 64 * ring + 5]                     # one in the first lap, one just after the ring has wrapped; never both in a window
    for j in big:
        h[j] = 60.0 * u                            # score 60 / 4 = 15 against about 0.25 for the others
    h = h.astype(np.float32).astype(np.float64)
    ref = P.causal_attention(h[:, None, :], h[:, None, :], h[:, None, :], window)[:, 0, :]
    e = attention_engine(torch.float32, part, h, max_tokens=1024)
    [_, a] = e.alloc(2)
    got = e.step([a], [range(n_prompt)])
    assert np.abs(got - ref[:n_prompt]).max() <= 1e-4
    assert len(e.engine.slot_pages(0, a)) <= ring
    for p in range(n_prompt, n_all):
        out = e.step([a], [[p]])[0]
        assert np.abs(out - ref[p]).max() <= 1e-4, p
        for j in big:
            if p == j + window - 1:
                assert out[3] > 50.0, (p, "the key at position - window + 1 is visible")
            if p == j + window:
                assert out[3] < 2.0, (p, "the key at position - window is dropped")
    assert len(e.engine.slot_pages(0, a)) == ring


# ------------------------------------------------------------------------------------------- parts with kernels of their own
class ToyConfig:
    def __init__(self, d):
        self.d = dict(d)
        self.hidden_size, self.vocab_size, self.intermediate_size = d["hidden_size"], d["vocab_size"], d["intermediate_size"]
        self.max_position_embeddings = d["max_position_embeddings"]
        self.torch_dtype = "bfloat16"
        self.eos_token_ids = ()

    def to_dict(self):
        return dict(self.d)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_parts_with_hip_kernels_of_their_own_run_in_the_engines_step(dtype, tmp_path):
    """A mixer with state of its own and a norm that is no RMSNorm, each a HIP kernel and a C
    function in a library beside the tests (tests/toy_parts).  Their parts, defined here, emit a
    called operation that names the C function; the engine hands it the running step.  Nothing
    of the library changes: the model is registered, built, loaded from a random folder and
    stepped through Session (prompts whole, from a cut token by token in reused slots, with decode
    steps that are recorded and replayed) and through the library's generation loop."""
    from toy_parts import build as toy_build
    from picolm_amd import SamplingParams
    from picolm_amd.config import register_architecture, unregister_architecture
    from picolm_amd.engine import DecoderModel, Session, load_model
    from picolm_amd.engine.program import Rows
    from picolm_amd.parts import LMHead, Mixer, Norm, PreNormBlock, RMSNorm, StateRequest, SwiGLU, TokenEmbedding
    from picolm_amd.weights import TensorSpec, write_random_model
    toy = toy_build.load()

    class MeanArgs(ctypes.Structure):
        _fields_ = [("w", ctypes.c_void_p), ("D", ctypes.c_int32), ("in_bf16", ctypes.c_int32)]

    class NormArgs(ctypes.Structure):
        _fields_ = [("w", ctypes.c_void_p), ("b", ctypes.c_void_p), ("D", ctypes.c_int32), ("eps", ctypes.c_float),
                    ("out_bf16", ctypes.c_int32)]

    class RunningMean(Mixer):
        def __init__(self, name, D):
            self.name, self.D, self.w = name, D, None

        def tensor_specs(self):
            return [TensorSpec(self.name, (self.D, self.D))]

        def load(self, fetch, runtime):
            self.w = fetch.get(self.name).float().contiguous()

        def cache_requests(self):
            return None, StateRequest((self.D + 1,), torch.float32)

        def emit(self, b, src, x, out_norm=None, out_norm_when=0):
            h = b.materialize(src)
            args = MeanArgs(self.w.data_ptr(), self.D, int(b.buffer_dtype(h) == torch.bfloat16))
            b.keep.append(self.w)
            b.call(toy.toy_running_mean, out=x, inp=h, user=args, uses_state=True, recordable=True)

    class CenteredNorm(Norm):
        def __init__(self, name, size, eps):
            self.name, self.size, self.eps = name, size, eps
            self.weight = self.bias = None

        def tensor_specs(self):
            return [TensorSpec(self.name + ".weight", (self.size,), init="ones"), TensorSpec(self.name + ".bias", (self.size,))]

        def load(self, fetch, runtime):
            self.weight = fetch.get(self.name + ".weight").float().contiguous()
            self.bias = fetch.get(self.name + ".bias").float().contiguous()

        def emit(self, b, x, rows=0):
            h = b.buffer("norm.final" if rows else "norm.out", self.size, b.dtype, rows)
            args = NormArgs(self.weight.data_ptr(), self.bias.data_ptr(), self.size, self.eps, int(b.dtype == torch.bfloat16))
            b.keep += [self.weight, self.bias]
            b.call(toy.toy_centered_norm, out=h, inp=x, rows=rows, user=args, recordable=True)
            return Rows(h)

    def build(cfg):
        D = cfg.hidden_size
        emb = TokenEmbedding("emb.weight", cfg.vocab_size, D)
        block = PreNormBlock(CenteredNorm("norm1", D, 1e-5), RunningMean("mean.weight", D),
                             RMSNorm("norm2.weight", D, 1e-5), SwiGLU("ffn.", D, cfg.intermediate_size))
        return DecoderModel(cfg, emb, [block], CenteredNorm("final", D, 1e-5),
                            LMHead("head.weight", cfg.vocab_size, D, emb, tied=True), order=[0, 0])

    name = "ToyKernelsLM"
    register_architecture(name, ToyConfig, build)
    try:
        cfg = ToyConfig(dict(architectures=[name], hidden_size=40, vocab_size=77, intermediate_size=56, max_position_embeddings=256))
        d = write_random_model(cfg, str(tmp_path / "toy"), seed=4, std=0.3)
        model = load_model(d, dtype=dtype)
        w = tiny.read_weights_f64(d)

        def centered(x, n):
            xc = x - x.mean(axis=1, keepdims=True)
            return xc / np.sqrt((xc * xc).mean(axis=1, keepdims=True) + 1e-5) * w[n + ".weight"] + w[n + ".bias"]

        def plain(tokens):
            x = w["emb.weight"][tokens]
            for _ in range(2):
                hh = centered(x, "norm1")
                mean = np.cumsum(hh, axis=0) / np.arange(1, len(tokens) + 1)[:, None]
                x = x + mean @ w["mean.weight"].T
                x = x + P.swiglu(P.rmsnorm(x, w["norm2.weight"], 1e-5), w["ffn.gate_proj.weight"],
                                 w["ffn.up_proj.weight"], w["ffn.down_proj.weight"])
            return centered(x, "final") @ w["emb.weight"].T
        rng = np.random.default_rng(7)
        reqs = [tiny.random_tokens(rng, n, 77) for n in (19, 3, 40)]
        truth = [plain(r) for r in reqs]
        bound = lambda t: tiny.tolerance(dtype, t, tiny.spread(40, 0.3)) * (1 if dtype == "float32" else 2)
        s = Session(model, max_tokens=512, n_slots=3)
        assert s.engine.program.recordable
        slots = s.begin(3)                                        # whole, as one unequal batch; some rows wanted, some not
        got = s.step(slots, reqs, [list(range(len(r))) for r in reqs]).double().cpu().numpy()
        row = 0
        for r, t in zip(reqs, truth):
            assert np.abs(got[row:row + len(r)] - t).max() <= bound(t)
            row += len(r)
        s.release(slots)
        slots = s.begin(3)                                        # reused slots: state starts from zero again
        cut = [7, 1, 33]
        got = s.step(slots, [r[:c] for r, c in zip(reqs, cut)], [[0], [], [5, 32]]).double().cpu().numpy()
        assert np.abs(got - np.stack([truth[0][0], truth[2][5], truth[2][32]])).max() <= bound(truth[2])
        pos = dict(zip(range(3), cut))
        live = [0, 1, 2]
        while live:
            out = s.step([slots[i] for i in live], [[reqs[i][pos[i]]] for i in live]).double().cpu().numpy()
            for k, i in enumerate(live):
                assert np.abs(out[k] - truth[i][pos[i]]).max() <= bound(truth[i]), (i, pos[i])
                pos[i] += 1
            live = [i for i in live if pos[i] < len(reqs[i])]
        assert s.recorded_steps() >= 2                            # three, two and one sequence: each shape recorded at its second use
        s.release(slots)
        if dtype == "float32":
            toks, finish = s.engine.generate([r[:5] for r in reqs], 6, SamplingParams(), [], batch_size=2)
            assert finish == ["length"] * 3
            for r, got in zip(reqs, toks):
                seq = list(r[:5])
                for t in got:
                    row = plain(np.asarray(seq))[-1]
                    assert row[t] >= row.max() - 1e-4
                    seq.append(t)
    finally:
        unregister_architecture(name)


def test_a_called_operation_that_fails_fails_the_step():
    """What a Python part raises inside the engine's step comes back to the step's caller as that
    exception; the sequences stay where they were."""
    from part_harness import PartEngine
    from picolm_amd.parts import FeedForward

    class Broken(FeedForward):
        def forward(self, ctx, h, residual):
            if ctx.batch.T > 3:
                raise ZeroDivisionError("more rows than this toy takes")
            residual += 1.0
    from picolm_amd.engine.program import Rows
    ffn = Broken()

    def emit(b, xb, h):
        ffn.emit(b, Rows(h.cast(b, xb, 8)), xb)
        return xb, 8
    e = PartEngine(torch.float32, np.zeros((6, 8), np.float32), emit, parts=[ffn])
    [a] = e.alloc(1)
    assert np.array_equal(e.step([a], [range(3)]), np.ones((3, 8)))
    with pytest.raises(ZeroDivisionError, match="more rows"):
        e.step([a], [range(4)])
    assert e.engine.length(a) == 3
    assert np.array_equal(e.step([a], [range(2)]), np.ones((2, 8)))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_subclasses_of_the_librarys_parts(dtype, tmp_path):
    """A subclass that changes a constant keeps the engine's own operations (and recorded decode
    steps); a subclass that changes `forward` runs through its `forward`.  Here: an attention with
    another scale, an RMSNorm whose weights are offset by a half, and a gated feed-forward whose
    output is halved."""
    from picolm_amd import LlamaConfig
    from picolm_amd.config import register_architecture, unregister_architecture
    from picolm_amd.engine import DecoderModel, Session, load_model
    from picolm_amd.engine.program import OP_CALL
    from picolm_amd.parts import Attention, LMHead, PreNormBlock, RMSNorm, RotaryEmbedding, SwiGLU, TokenEmbedding
    from picolm_amd.weights import write_random_model

    class SharpAttention(Attention):
        def __init__(self, *a, **kw):
            super().__init__(*a, **kw)
            self.scale *= 1.5

    class OffsetNorm(RMSNorm):
        def __init__(self, name, size, eps):
            super().__init__(name, size, eps, weight_offset=0.5)

    class HalvedSwiGLU(SwiGLU):
        def forward(self, ctx, h, residual):
            out = torch.zeros_like(residual)
            super().forward(ctx, h, out)
            residual += 0.5 * out

    def build(cfg, halved=True):
        D = cfg.hidden_size
        rotary = RotaryEmbedding(cfg.head_dim, cfg.rope_theta, None, cfg.rope_style)
        blocks = []
        for l in range(2):
            q = f"model.layers.{l}."
            ffn = (HalvedSwiGLU if halved and l == 1 else SwiGLU)(q + "mlp.", D, cfg.intermediate_size)
            blocks.append(PreNormBlock(OffsetNorm(q + "input_layernorm.weight", D, cfg.rms_norm_eps),
                                       SharpAttention(q + "self_attn.", D, cfg.num_attention_heads, cfg.num_key_value_heads,
                                                      cfg.head_dim, position=rotary),
                                       RMSNorm(q + "post_attention_layernorm.weight", D, cfg.rms_norm_eps), ffn))
        emb = TokenEmbedding("model.embed_tokens.weight", cfg.vocab_size, D)
        return DecoderModel(cfg, emb, blocks, RMSNorm("model.norm.weight", D, cfg.rms_norm_eps),
                            LMHead("lm_head.weight", cfg.vocab_size, D, emb, True))

    c = dict(architectures=["ToySubclassLM"], hidden_size=128, num_attention_heads=4, num_key_value_heads=2, head_dim=32,
             intermediate_size=192, num_hidden_layers=2, vocab_size=211, rms_norm_eps=1e-5, rope_theta=10000.0,
             max_position_embeddings=256, tie_word_embeddings=True, torch_dtype="bfloat16")
    cfg = LlamaConfig.from_dict(c)
    register_architecture("ToySubclassLM", LlamaConfig.from_dict, build)
    try:
        d = write_random_model(cfg, str(tmp_path / "sub"), seed=5, std=0.08)
    finally:
        unregister_architecture("ToySubclassLM")
    w = tiny.read_weights_f64(d)
    pc = dict(c, rope_style=cfg.rope_style)

    def plain(tokens, halved):
        pos = np.arange(len(tokens))
        x = w["model.embed_tokens.weight"][np.asarray(tokens)]
        for l in range(2):
            q = f"model.layers.{l}."
            h = P.rmsnorm(x, w[q + "input_layernorm.weight"] + 0.5, 1e-5)
            sharp = {k: (v * 1.5 if k == q + "self_attn.q_proj.weight" else v) for k, v in w.items() if k.startswith(q)}
            x = x + P.attention_block(h, sharp, q + "self_attn.", pc, pos)      # (a scale on the scores is a scale on q)
            h = P.rmsnorm(x, w[q + "post_attention_layernorm.weight"], 1e-5)
            y = P.swiglu(h, w[q + "mlp.gate_proj.weight"], w[q + "mlp.up_proj.weight"], w[q + "mlp.down_proj.weight"])
            x = x + (0.5 * y if halved and l == 1 else y)
        return P.rmsnorm(x, w["model.norm.weight"], 1e-5) @ w["model.embed_tokens.weight"].T
    rng = np.random.default_rng(9)
    reqs = [tiny.random_tokens(rng, n, 211) for n in (70, 5, 33)]
    for halved in (False, True):
        register_architecture("ToySubclassLM", LlamaConfig.from_dict, lambda cf: build(cf, halved))
        try:
            model = load_model(d, dtype=dtype)
        finally:
            unregister_architecture("ToySubclassLM")
        truth = [plain(r, halved) for r in reqs]
        tol_ = lambda t: tiny.tolerance(dtype, t, tiny.spread(128, 0.08))
        s = Session(model, max_tokens=512, n_slots=3)
        assert sum(op.kind == OP_CALL for op in s.engine.program.ops) == int(halved)       # only the changed forward is a call
        slots = s.begin(3)
        cut = [50, 2, 20]
        s.step(slots, [r[:c_] for r, c_ in zip(reqs, cut)])
        pos, live = dict(zip(range(3), cut)), [0, 1, 2]
        while live:
            out = s.step([slots[i] for i in live], [[reqs[i][pos[i]]] for i in live]).double().cpu().numpy()
            for k, i in enumerate(live):
                assert np.abs(out[k] - truth[i][pos[i]]).max() <= tol_(truth[i]), (halved, i, pos[i])
                pos[i] += 1
            live = [i for i in live if pos[i] < len(reqs[i])]
        assert (s.recorded_steps() > 0) == (not halved)


def test_a_prepared_norm_is_forgotten_when_its_rows_are_written_again():
    """A product that adds into the residual rows may prepare the norm that meets them next.  If
    another operation writes those rows before the norm is taken (two branches that add into the
    stream one after the other), what was prepared describes rows that are no more: the product that
    takes the norm must see the rows as they are.  Few rows, where the products share norms."""
    from part_harness import PartEngine
    from picolm_amd import kernels as K
    from picolm_amd.engine.program import NormRef, Rows
    rng = np.random.default_rng(12)
    D, T = 256, 5
    x0 = rounded(rng.standard_normal((T, D)), torch.bfloat16)
    w = {n: rounded(rng.standard_normal((D, D)) * 0.05, torch.bfloat16) for n in ("w1", "w2", "w3")}
    nw = rng.standard_normal(D)
    dev = {n: torch.from_numpy(v).to(torch.bfloat16).to(DEV) for n, v in w.items()}
    norm = NormRef(torch.from_numpy(nw).float().to(DEV), 1e-5)

    def emit(b, x, h):
        hb = h.cast(b, x, D)
        b.linear(dev["w1"], hb, x, K.EPI_ACCUMULATE, out_norm=norm)       # prepares norm(x) where its kernel can
        b.linear(dev["w2"], hb, x, K.EPI_ACCUMULATE)                       # and x changes again
        y = b.buffer("y", D, torch.float32)
        b.linear(dev["w3"], Rows(b.buffer("norm.out", D, torch.bfloat16), norm, x), y, K.EPI_STORE)
        return y, D
    e = PartEngine(torch.bfloat16, x0, emit)
    got = e.step(e.alloc(1), [range(T)])
    x = x0 + x0 @ w["w1"].T + x0 @ w["w2"].T
    ref = P.rmsnorm(x, nw.astype(np.float32), 1e-5) @ w["w3"].T
    stale = P.rmsnorm(x0 + x0 @ w["w1"].T, nw.astype(np.float32), 1e-5) @ w["w3"].T
    assert np.abs(ref - stale).max() > 20 * tol(torch.bfloat16, ref)          # the fault would show
    assert np.abs(got - ref).max() <= tol(torch.bfloat16, ref)


def test_a_python_part_that_says_graph_safe_is_recorded_and_replayed(tmp_path):
    """A feed-forward written in Python whose `forward` only launches the library's kernels on
    buffers that exist after its first use, and says so (`graph_safe = True`): the decode steps of
    its model are recorded on the engine's own stream and replayed, and give the bits of steps that
    are launched one by one, and the plain implementation's logits."""
    from picolm_amd import LlamaConfig
    from picolm_amd import kernels as K
    from picolm_amd.config import register_architecture, unregister_architecture
    from picolm_amd.engine import DecoderModel, Session, load_model
    from picolm_amd.parts import (Attention, FeedForward, Linear, LMHead, PreNormBlock, RMSNorm, RotaryEmbedding, TokenEmbedding)
    from picolm_amd.weights import write_random_model

    class TwoProducts(FeedForward):
        """down(up(h)): no gate, no activation"""
        graph_safe = True

        def __init__(self, prefix, D, F):
            self.F = F
            self.up = Linear([prefix + "up_proj.weight"], [F], D)
            self.down = Linear([prefix + "down_proj.weight"], [D], F)

        def children(self):
            return [self.up, self.down]

        def forward(self, ctx, h, residual):
            act = ctx.ws.get("toy.act", (h.shape[0], self.F), ctx.dtype)
            self.up.forward(h, act)
            self.down.forward(act, residual, K.EPI_ACCUMULATE)

    def build(cfg):
        D = cfg.hidden_size
        rotary = RotaryEmbedding(cfg.head_dim, cfg.rope_theta, None, cfg.rope_style)
        blocks = [PreNormBlock(RMSNorm(f"model.layers.{l}.input_layernorm.weight", D, cfg.rms_norm_eps),
                               Attention(f"model.layers.{l}.self_attn.", D, cfg.num_attention_heads, cfg.num_key_value_heads,
                                         cfg.head_dim, position=rotary),
                               RMSNorm(f"model.layers.{l}.post_attention_layernorm.weight", D, cfg.rms_norm_eps),
                               TwoProducts(f"model.layers.{l}.mlp.", D, cfg.intermediate_size)) for l in range(2)]
        emb = TokenEmbedding("model.embed_tokens.weight", cfg.vocab_size, D)
        return DecoderModel(cfg, emb, blocks, RMSNorm("model.norm.weight", D, cfg.rms_norm_eps),
                            LMHead("lm_head.weight", cfg.vocab_size, D, emb, True))

    name = "ToyTwoProductsLM"
    c = dict(architectures=[name], hidden_size=128, num_attention_heads=4, num_key_value_heads=2, head_dim=32,
             intermediate_size=192, num_hidden_layers=2, vocab_size=211, rms_norm_eps=1e-5, rope_theta=10000.0,
             max_position_embeddings=256, tie_word_embeddings=True, torch_dtype="bfloat16")
    cfg = LlamaConfig.from_dict(c)
    register_architecture(name, LlamaConfig.from_dict, build)
    try:
        d = write_random_model(cfg, str(tmp_path / "two"), seed=6, std=0.08)
        model = load_model(d, dtype="bfloat16")
    finally:
        unregister_architecture(name)
    w = tiny.read_weights_f64(d)
    pc = dict(c, rope_style=cfg.rope_style)

    def plain(tokens):
        pos = np.arange(len(tokens))
        x = w["model.embed_tokens.weight"][np.asarray(tokens)]
        for l in range(2):
            q = f"model.layers.{l}."
            x = x + P.attention_block(P.rmsnorm(x, w[q + "input_layernorm.weight"], 1e-5), w, q + "self_attn.", pc, pos)
            h = P.rmsnorm(x, w[q + "post_attention_layernorm.weight"], 1e-5)
            x = x + (h @ w[q + "mlp.up_proj.weight"].T) @ w[q + "mlp.down_proj.weight"].T
        return P.rmsnorm(x, w["model.norm.weight"], 1e-5) @ w["model.embed_tokens.weight"].T
    rng = np.random.default_rng(10)
    reqs = [tiny.random_tokens(rng, n, 211) for n in (40, 9)]
    truth = [plain(r) for r in reqs]
    outs = []
    for graphs in (True, False):
        s = Session(model, max_tokens=512, n_slots=2, graphs=graphs)
        assert s.engine.program.recordable
        slots = s.begin(2)
        rows = [s.step(slots, [r[:5] for r in reqs]).clone()]
        for j in range(5, 9):
            rows.append(s.step(slots, [[r[j]] for r in reqs]).clone())
        assert (s.recorded_steps() == 1) == graphs
        outs.append(rows)
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    for j, row in enumerate(outs[0]):
        for i in range(2):
            ref = truth[i][4 + j]
            assert np.abs(row[i].double().cpu().numpy() - ref).max() <= tiny.tolerance("bfloat16", truth[i], tiny.spread(128, 0.08))


def test_a_toy_mixer_over_a_window_takes_long_prompts_in_steps_that_fit_its_ring(tmp_path):
    """A one-head attention with a window of 40 keys, defined here and run as a called operation
    on a group that keeps a ring of pages.  The attention operation answers a long prompt over a
    ring slice by slice; a called operation sees its step whole, so the engine refuses a step of
    more than 256 tokens a sequence, says how many a step may bring, and both generation loops cut
    the prompts accordingly: their tokens are those of the plain model with the same window."""
    from picolm_amd import SamplingParams
    from picolm_amd.cache import PAGE_TOKENS, window_ring_pages
    from picolm_amd.config import register_architecture, unregister_architecture
    from picolm_amd.engine import DecoderModel, Session, StepError, load_model
    from picolm_amd.generation import generate
    from picolm_amd.parts import KVRequest, LMHead, Mixer, PreNormBlock, RMSNorm, SwiGLU, TokenEmbedding
    from picolm_amd.weights import TensorSpec, write_random_model
    DK, WINDOW = 16, 40

    class ToyConfig:
        def __init__(self, d):
            self.d = dict(d)
            self.hidden_size, self.vocab_size, self.intermediate_size = d["hidden_size"], d["vocab_size"], d["intermediate_size"]
            self.max_position_embeddings = d["max_position_embeddings"]
            self.torch_dtype = "bfloat16"
            self.eos_token_ids = ()

        def to_dict(self):
            return dict(self.d)

    class NearKeys(Mixer):
        def __init__(self, prefix, D):
            self.prefix, self.D, self.w = prefix, D, {}

        def tensor_specs(self):
            return [TensorSpec(self.prefix + c, (DK, self.D)) for c in "qkv"] + [TensorSpec(self.prefix + "o", (self.D, DK))]

        def load(self, fetch, runtime):
            self.w = {n: fetch.get(self.prefix + n).float() for n in "qkvo"}

        def cache_requests(self):
            return KVRequest(1, DK, WINDOW), None

        def forward(self, ctx, h, residual):
            k_pages, v_pages, table, ring = ctx.kv()
            assert ring == window_ring_pages(WINDOW) < table.shape[1]
            b, row = ctx.batch, 0
            for slot, p0, n in zip(b.slots, b.pos0, b.n_new):
                x = h[row:row + n].float()
                q, k, v = x @ self.w["q"].T, x @ self.w["k"].T, x @ self.w["v"].T
                lo = max(0, p0 - WINDOW + 1)                              # the oldest key that any of the new queries sees
                pos = torch.arange(lo, p0 + n, device=x.device)
                page, at = table[slot, (pos // PAGE_TOKENS) % ring].long(), pos % PAGE_TOKENS
                new = slice(p0 - lo, None)
                k_pages[page[new], 0, at[new]] = k.to(k_pages.dtype)
                v_pages[page[new], 0, :, at[new]] = v.to(v_pages.dtype)
                keys, values = k_pages[page, 0, at].float(), v_pages[page, 0, :, at].float()
                s = q @ keys.T / math.sqrt(DK)
                hidden = (pos[None, :] > pos[new, None]) | (pos[new, None] - pos[None, :] >= WINDOW)
                residual[row:row + n] += (torch.softmax(s.masked_fill(hidden, float("-inf")), dim=-1) @ values) @ self.w["o"].T
                row += n

    def build(cfg):
        D = cfg.hidden_size
        emb = TokenEmbedding("emb.weight", cfg.vocab_size, D)
        blocks = [PreNormBlock(RMSNorm(f"l{i}.norm1.weight", D, 1e-5), NearKeys(f"l{i}.mix.", D),
                               RMSNorm(f"l{i}.norm2.weight", D, 1e-5), SwiGLU(f"l{i}.ffn.", D, cfg.intermediate_size)) for i in range(2)]
        return DecoderModel(cfg, emb, blocks, RMSNorm("final.weight", D, 1e-5),
                            LMHead("head.weight", cfg.vocab_size, D, emb, tied=True))

    register_architecture("ToyNearKeysLM", ToyConfig, build)
    try:
        cfg = ToyConfig(dict(architectures=["ToyNearKeysLM"], hidden_size=40, vocab_size=77, intermediate_size=56,
                             max_position_embeddings=1024))
        d = write_random_model(cfg, str(tmp_path / "toy"), seed=6, std=0.3)
        model = load_model(d, dtype="float32")
        w = tiny.read_weights_f64(d)

        def plain(tokens):
            x = w["emb.weight"][tokens]
            n = len(tokens)
            far = np.arange(n)[:, None] - np.arange(n)[None, :]
            for i in range(2):
                hh = P.rmsnorm(x, w[f"l{i}.norm1.weight"], 1e-5)
                q, k, v = (hh @ w[f"l{i}.mix.{c}"].T for c in "qkv")
                s = q @ k.T / math.sqrt(DK)
                s[(far < 0) | (far >= WINDOW)] = -np.inf
                p = np.exp(s - s.max(axis=1, keepdims=True))
                x = x + (p / p.sum(axis=1, keepdims=True)) @ v @ w[f"l{i}.mix.o"].T
                x = x + P.swiglu(P.rmsnorm(x, w[f"l{i}.norm2.weight"], 1e-5), w[f"l{i}.ffn.gate_proj.weight"],
                                 w[f"l{i}.ffn.up_proj.weight"], w[f"l{i}.ffn.down_proj.weight"])
            return P.rmsnorm(x, w["final.weight"], 1e-5) @ w["emb.weight"].T

        def plain_greedy(prompt, n_new):
            toks = list(prompt)
            for _ in range(n_new):
                toks.append(int(np.argmax(plain(toks)[-1])))
            return toks[len(prompt):]
        rng = np.random.default_rng(12)
        reqs = [tiny.random_tokens(rng, n, 77) for n in (300, 20, 600)]
        s = Session(model, max_tokens=2048, n_slots=3)
        assert s.most_new_tokens == 256
        slots = s.begin(3)
        with pytest.raises(StepError, match="up to 256 tokens a sequence, sequence 0 brings 300"):
            s.step(slots, reqs)
        assert [s.length(x) for x in slots] == [0, 0, 0]
        # whole prompts in steps that fit, every position against the plain model
        got = [[], [], []]
        for lo in range(0, 600, 256):
            live = [i for i in range(3) if len(reqs[i]) > lo]
            out = s.step([slots[i] for i in live], [reqs[i][lo:lo + 256] for i in live],
                         [list(range(len(reqs[i][lo:lo + 256]))) for i in live]).double().cpu().numpy()
            for i in live:
                n = len(reqs[i][lo:lo + 256])
                got[i].append(out[:n])
                out = out[n:]
        for i in range(3):
            assert np.abs(np.concatenate(got[i]) - plain(reqs[i])).max() < 1e-4, i
        s.release(slots)
        want = [plain_greedy(r, 6) for r in reqs]
        outs = generate(s, reqs, max_new_tokens=6, params=SamplingParams(temperature=0.0), stop_ids=(), batch_size=3)
        assert [o.tokens for o in outs] == want
        tokens, reasons = s.engine.generate(reqs, 6, SamplingParams(temperature=0.0), (), batch_size=3)
        assert tokens == want and reasons == ["length"] * 3
    finally:
        unregister_architecture("ToyNearKeysLM")


TOY_ARCHITECTURE_MODULE = '''
"""An architecture outside the package: a decoder whose mixer is the running mean of its inputs,
kept as state per sequence.  Importing the module registers it."""
import torch

from picolm_amd.config import register_architecture
from picolm_amd.engine import DecoderModel
from picolm_amd.parts import LMHead, Mixer, PreNormBlock, RMSNorm, StateRequest, SwiGLU, TokenEmbedding
from picolm_amd.weights import TensorSpec


class Config:
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
        state, b, row = ctx.state(), ctx.batch, 0
        for slot, n in zip(b.slots, b.n_new):
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
    return DecoderModel(cfg, emb, [block], RMSNorm("final.weight", D, 1e-5), LMHead("head.weight", cfg.vocab_size, D, emb, tied=True))


register_architecture("ToyOutsideLM", Config, build)
'''


def test_an_architecture_from_a_module_outside_the_package_runs_through_the_programs(tmp_path):
    """The module above lies in a folder of its own.  With that folder on the module path and the
    module's name in PICOLM_ARCHITECTURES, `bin/trace_run` and `bin/picolm` load a model of that
    architecture, step it and generate with it, with no file of the package changed: the replayed
    logits are those of a session in this process and of the plain form of the model."""
    import subprocess
    import sys
    from picolm_amd.config import import_architecture_modules, unregister_architecture
    from picolm_amd.engine import Session, load_model
    from picolm_amd.weights import write_random_model
    from replay_util import ROOT, TraceRun
    folder = tmp_path / "outside"
    folder.mkdir()
    (folder / "toy_outside_arch.py").write_text(TOY_ARCHITECTURE_MODULE)
    env = dict(os.environ, PICOLM_ARCHITECTURES="toy_outside_arch",
               PYTHONPATH=os.pathsep.join([str(folder)] + [p for p in [os.environ.get("PYTHONPATH")] if p]))
    sys.path.insert(0, str(folder))
    try:
        assert import_architecture_modules("toy_outside_arch") == ["toy_outside_arch"]
        import toy_outside_arch
        cfg = toy_outside_arch.Config(dict(architectures=["ToyOutsideLM"], hidden_size=40, vocab_size=77, intermediate_size=56,
                                           max_position_embeddings=256))
        d = write_random_model(cfg, str(tmp_path / "toy"), seed=14, std=0.3)
        w = tiny.read_weights_f64(d)

        def plain(tokens):
            x = w["emb.weight"][tokens]
            hh = P.rmsnorm(x, w["norm1.weight"], 1e-5)
            x = x + (np.cumsum(hh, axis=0) / np.arange(1, len(tokens) + 1)[:, None]) @ w["mean.weight"].T
            x = x + P.swiglu(P.rmsnorm(x, w["norm2.weight"], 1e-5), w["ffn.gate_proj.weight"], w["ffn.up_proj.weight"],
                             w["ffn.down_proj.weight"])
            return P.rmsnorm(x, w["final.weight"], 1e-5) @ w["emb.weight"].T
        rng = np.random.default_rng(3)
        a, b = tiny.random_tokens(rng, 30, 77), tiny.random_tokens(rng, 9, 77)
        tr = TraceRun(d, "float32", str(tmp_path / "out"), 256, env=env)
        got = tr.step([("a", a[:25], [0, 24]), ("b", b[:8], [7])])
        assert np.abs(got - np.stack([plain(a)[0], plain(a)[24], plain(b)[7]])).max() < 5e-5
        got = tr.step([("a", [a[25]], [0]), ("b", [b[8]], [0])], end=["b"])
        assert np.abs(got - np.stack([plain(a)[25], plain(b)[8]])).max() < 5e-5
        got = tr.step([("a", [a[26]], [0])], end=["a"])
        assert np.abs(got[0] - plain(a)[26]).max() < 5e-5
        tr.close()
        # the command line generates with it: greedy tokens as a session in this process gives them
        s = Session(load_model(d, dtype="float32"), max_tokens=256)
        [slot] = s.begin(1)
        seq = list(a[:12])
        row = s.step([slot], [seq])[0]
        want = []
        for _ in range(5):
            want.append(int(torch.argmax(row)))
            row = s.step([slot], [[want[-1]]])[0]
        out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "picolm"), d, "-p", " ".join(map(str, a[:12])), "-n", "5",
                              "-t", "0", "--dtype", "float32"], env=env, capture_output=True, text=True, timeout=300)
        assert out.returncode == 0, out.stderr
        assert [int(t) for t in out.stdout.split()] == want
        # without the variable the name is unknown, and the message says which names are known
        bare = dict(env)
        del bare["PICOLM_ARCHITECTURES"]
        out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "picolm"), d, "-p", "1 2", "-n", "1"], env=bare,
                             capture_output=True, text=True, timeout=300)
        assert out.returncode != 0 and "ToyOutsideLM" in out.stderr and "LlamaForCausalLM" in out.stderr
    finally:
        sys.path.remove(str(folder))
        sys.modules.pop("toy_outside_arch", None)
        unregister_architecture("ToyOutsideLM")
