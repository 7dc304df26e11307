"""What pins the plain implementation beside the reference's text: special cases that reduce
to a library routine, invariants, and hand-computed values.  Each is chosen so that a plausible
mistake (a wrong sign or pairing, a norm in the wrong place, an off-by-one mask) fails it.
The reference's own tests hold no vector for these parts (its one unit test is about quantised
dot products), so parity with its compiled output is unpinned; its formulas are."""
import math

import numpy as np
import pytest
import torch

import tiny
from plain import llama_plain as P
from plain import sampler_plain as SP


# ---------------------------------------------------------------------------------------- norm
def test_rmsnorm_formula_and_invariants():
    rng = np.random.default_rng(0)
    x, w = rng.standard_normal((3, 40)), rng.standard_normal(40)
    want = x / np.sqrt((x ** 2).mean(-1, keepdims=True) + 1e-5) * w
    assert np.allclose(P.rmsnorm(x, w, 1e-5), want, rtol=1e-12)
    y = P.rmsnorm(x, np.ones(40), 0.0)
    assert np.allclose(np.sqrt((y ** 2).mean(-1)), 1.0)                 # unit RMS
    assert np.allclose(P.rmsnorm(5.0 * x, w, 0.0), P.rmsnorm(x, w, 0.0))  # scale invariance at eps = 0
    assert not np.allclose(P.rmsnorm(x + 1.0, np.ones(40), 0.0).mean(-1), 0.0)   # no mean is subtracted
    # eps sits inside the root, added to the mean (not to the sum, not outside the root)
    one = P.rmsnorm(np.full((1, 4), 2.0), np.ones(4), 5.0)
    assert np.allclose(one, 2.0 / math.sqrt(4.0 + 5.0))


# ---------------------------------------------------------------------------------------- rope
def test_rope_tables_and_identity_at_position_zero():
    inv = P.rope_inv_freq(8, 10000.0)
    assert np.allclose(inv, [1.0, 10000 ** -0.25, 10000 ** -0.5, 10000 ** -0.75])
    cos, sin = P.rope_tables(np.array([0, 3]), inv)
    assert np.allclose(cos[0], 1) and np.allclose(sin[0], 0)
    assert np.allclose(cos[1], np.cos(3 * inv)) and np.allclose(sin[1], np.sin(3 * inv))
    x = np.random.default_rng(1).standard_normal((2, 3, 8))
    for style in ("pairwise", "half"):
        assert np.allclose(P.apply_rope(x, cos, sin, style)[0], x[0])


@pytest.mark.parametrize("style", ["pairwise", "half"])
def test_rope_is_a_rotation_by_plus_theta(style):
    # the pair (1, 0) at angle t becomes (cos t, sin t): fixes the sign of the sine terms
    d = 4
    inv = np.array([0.5, 0.25])
    cos, sin = P.rope_tables(np.array([2]), inv)
    x = np.zeros((1, 1, d))
    i0, i1 = (0, 1) if style == "pairwise" else (0, 2)
    x[0, 0, i0] = 1.0
    y = P.apply_rope(x, cos, sin, style)[0, 0]
    assert np.isclose(y[i0], math.cos(1.0)) and np.isclose(y[i1], math.sin(1.0))
    # norms of pairs are kept
    z = np.random.default_rng(2).standard_normal((1, 2, d))
    r = P.apply_rope(z, cos, sin, style)
    assert np.allclose((r ** 2).sum(-1), (z ** 2).sum(-1))


@pytest.mark.parametrize("style", ["pairwise", "half"])
def test_rope_scores_depend_on_distance_only(style):
    rng = np.random.default_rng(3)
    d = 16
    inv = P.rope_inv_freq(d, 500.0)
    q, k = rng.standard_normal((1, 1, d)), rng.standard_normal((1, 1, d))

    def score(m, n):
        cq, sq = P.rope_tables(np.array([m]), inv)
        ck, sk = P.rope_tables(np.array([n]), inv)
        return float((P.apply_rope(q, cq, sq, style) * P.apply_rope(k, ck, sk, style)).sum())
    assert np.isclose(score(7, 3), score(107, 103))
    assert np.isclose(score(7, 3), score(4, 0))
    assert not np.isclose(score(7, 3), score(3, 7))        # direction matters


def test_pairwise_and_half_agree_after_permuting_the_head():
    rng = np.random.default_rng(4)
    d = 8
    perm = np.concatenate([np.arange(0, d, 2), np.arange(1, d, 2)])     # pairwise layout -> half layout
    inv = P.rope_inv_freq(d, 100.0)
    cos, sin = P.rope_tables(np.arange(5), inv)
    x = rng.standard_normal((5, 2, d))
    assert np.allclose(P.apply_rope(x, cos, sin, "pairwise")[..., perm], P.apply_rope(x[..., perm], cos, sin, "half"))


def test_llama3_scaling_properties():
    sc = dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=64)
    base = P.rope_inv_freq(32, 500000.0)
    s = P.rope_inv_freq(32, 500000.0, sc)
    wl = 2 * math.pi / base
    assert np.allclose(s[wl < 16], base[wl < 16])                       # short wavelengths are kept
    assert np.allclose(s[wl > 64], base[wl > 64] / 8)                   # long ones divided by the factor
    mid = (wl >= 16) & (wl <= 64)
    assert mid.any() and np.all(s[mid] <= base[mid] + 1e-15) and np.all(s[mid] >= base[mid] / 8 - 1e-15)
    assert np.all(np.diff(s) < 0)                                       # still decreasing in i
    assert np.allclose(P.rope_inv_freq(32, 500000.0, dict(sc, factor=1.0)), base)
    # continuous at both thresholds: the blend weight is 1 at wavelength orig/high and 0 at orig/low
    for edge, want in ((16.0, 1.0), (64.0, 1 / 8)):
        smooth = (64 / edge - 1.0) / 3.0
        assert np.isclose((1 - smooth) / 8 + smooth, want)
    # and the scaled frequency itself does not jump there: head size 4 has f_1 = theta^(-1/2),
    # so theta = (wavelength / 2 pi)^2 puts f_1 at any wavelength
    def scaled_over_base(wavelength):
        theta = (wavelength / (2 * math.pi)) ** 2
        return P.rope_inv_freq(4, theta, sc)[1] / P.rope_inv_freq(4, theta)[1]
    for edge in (16.0, 64.0):
        assert abs(scaled_over_base(edge * (1 - 1e-9)) - scaled_over_base(edge * (1 + 1e-9))) < 1e-6
    assert np.isclose(scaled_over_base(10.0), 1.0) and np.isclose(scaled_over_base(100.0), 1 / 8)
    assert 1 / 8 < scaled_over_base(32.0) < 1.0
    # the blend is linear in original/wavelength, not in the wavelength: at wavelength 32 that ratio
    # is 2, a third of the way from low = 1 to high = 4, so the weight of the unscaled frequency
    # is 1/3 and the result (2/3)/8 + 1/3 = 5/12; a blend linear in the wavelength would weigh it
    # (64 - 32) / (64 - 16) = 2/3 and give 17/24
    assert np.isclose(scaled_over_base(32.0), 5 / 12, rtol=1e-12)
    assert np.isclose(scaled_over_base(48.0), (1 - 1 / 9) / 8 + 1 / 9, rtol=1e-12)      # ratio 4/3: weight 1/9


def test_the_engine_tables_use_the_same_frequencies():
    # the product's own routine (it runs on the host) against the plain one and the hand value
    from picolm_amd.config import LlamaConfig
    from picolm_amd.parts.position import rotary_inv_freq
    cfg = LlamaConfig.from_dict(dict(tiny.TINY_B))
    got = rotary_inv_freq(32, 500000.0, cfg.rope_scaling).numpy()
    want = P.rope_inv_freq(32, 500000.0, tiny.TINY_B["rope_scaling"])
    assert np.allclose(got, want, rtol=1e-14)
    theta = (32.0 / (2 * math.pi)) ** 2
    assert np.isclose(float(rotary_inv_freq(4, theta, cfg.rope_scaling)[1] / rotary_inv_freq(4, theta)[1]), 5 / 12, rtol=1e-12)


# ---------------------------------------------------------------------------------------- attention
def test_attention_equals_the_library_routine():
    rng = np.random.default_rng(5)
    T, H, d = 9, 3, 8
    q, k, v = (rng.standard_normal((T, H, d)) for _ in range(3))
    want = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q).permute(1, 0, 2), torch.from_numpy(k).permute(1, 0, 2), torch.from_numpy(v).permute(1, 0, 2),
        is_causal=True).permute(1, 0, 2).numpy()
    assert np.allclose(P.causal_attention(q, k, v), want, atol=1e-12)


def test_attention_special_cases():
    rng = np.random.default_rng(6)
    T, H, G, d = 6, 4, 2, 8
    q, k, v = rng.standard_normal((T, H, d)), rng.standard_normal((T, G, d)), rng.standard_normal((T, G, d))
    out = P.causal_attention(q, k, v)
    assert np.allclose(out[0, 0], v[0, 0]) and np.allclose(out[0, 3], v[0, 1])      # one key: its value row; head h reads group h // 2
    assert np.allclose(P.causal_attention(np.zeros_like(q), k, v)[3, 0], v[:4, 0].mean(0))   # equal scores: the mean
    rep = P.causal_attention(q, np.repeat(k, 2, axis=1), np.repeat(v, 2, axis=1))
    assert np.allclose(out, rep)                                                   # GQA = MHA with repeated KV heads
    # the future is not seen: changing a later key changes nothing earlier
    k2, v2 = k.copy(), v.copy()
    k2[4:], v2[4:] = 9.0, -9.0
    assert np.allclose(P.causal_attention(q, k2, v2)[:4], out[:4])
    # a window of w keys: position p sees p-w+1..p
    w = P.causal_attention(q, k, v, window=2)
    assert np.allclose(w[:2], out[:2]) and not np.allclose(w[3], out[3])
    assert np.allclose(w[5, 0], P.causal_attention(q[4:], k[4:], v[4:])[1, 0])
    # scale is 1/sqrt(d): one dominating key at score s*s/sqrt(d)
    qq, kk, vv = np.zeros((2, 1, 4)), np.zeros((2, 1, 4)), np.eye(2)[:, None, :].repeat(2, axis=2)
    qq[1, 0, 0], kk[0, 0, 0] = 2.0, 2.0
    p0 = math.exp(4 / 2.0) / (math.exp(4 / 2.0) + 1.0)
    assert np.allclose(P.causal_attention(qq, kk, vv)[1, 0, 0], p0)


# ---------------------------------------------------------------------------------------- ffn, model
def test_swiglu():
    rng = np.random.default_rng(7)
    x = rng.standard_normal((4, 6))
    wg, wu, wd = rng.standard_normal((10, 6)), rng.standard_normal((10, 6)), rng.standard_normal((6, 10))
    want = (torch.nn.functional.silu(torch.from_numpy(x @ wg.T)).numpy() * (x @ wu.T)) @ wd.T
    assert np.allclose(P.swiglu(x, wg, wu, wd), want)
    assert np.allclose(P.swiglu(x, np.zeros_like(wg), wu, wd), 0.0)     # gate 0 -> output 0
    assert np.isclose(P.silu(np.array([1.0]))[0], 1 / (1 + math.exp(-1)))


def small_model(tied):
    rng = np.random.default_rng(8)
    cfg = dict(num_hidden_layers=1, num_attention_heads=2, num_key_value_heads=1, head_dim=4, rms_norm_eps=1e-5,
               rope_theta=100.0)
    D, F, V = 6, 5, 11
    w = {"model.embed_tokens.weight": rng.standard_normal((V, D)), "model.norm.weight": rng.standard_normal(D),
         "model.layers.0.input_layernorm.weight": rng.standard_normal(D),
         "model.layers.0.post_attention_layernorm.weight": rng.standard_normal(D),
         "model.layers.0.self_attn.q_proj.weight": rng.standard_normal((8, D)),
         "model.layers.0.self_attn.k_proj.weight": rng.standard_normal((4, D)),
         "model.layers.0.self_attn.v_proj.weight": rng.standard_normal((4, D)),
         "model.layers.0.self_attn.o_proj.weight": rng.standard_normal((D, 8)),
         "model.layers.0.mlp.gate_proj.weight": rng.standard_normal((F, D)),
         "model.layers.0.mlp.up_proj.weight": rng.standard_normal((F, D)),
         "model.layers.0.mlp.down_proj.weight": rng.standard_normal((D, F))}
    if not tied:
        w["lm_head.weight"] = rng.standard_normal((V, D))
    return cfg, w


def test_whole_model_structure():
    cfg, w = small_model(tied=True)
    toks = [3, 1, 4, 1, 5]
    full = P.forward(w, cfg, toks)
    assert full.shape == (5, 11)
    assert np.allclose(P.forward(w, cfg, toks[:3]), full[:3])           # causal: a prefix gives the same rows
    assert np.allclose(full[1], P.forward(w, cfg, [3, 1])[-1])
    # the residual stream: with zero output projections the model is embedding -> final norm -> head
    w0 = dict(w)
    w0["model.layers.0.self_attn.o_proj.weight"] = np.zeros((6, 8))
    w0["model.layers.0.mlp.down_proj.weight"] = np.zeros((6, 5))
    e = w["model.embed_tokens.weight"]
    want = P.rmsnorm(e[toks], w["model.norm.weight"], 1e-5) @ e.T        # tied head = embedding table
    assert np.allclose(P.forward(w0, cfg, toks), want)
    cfg2, w2 = small_model(tied=False)
    a = P.forward(w2, cfg2, toks)
    w2b = dict(w2, **{"lm_head.weight": 2 * w2["lm_head.weight"]})
    assert np.allclose(P.forward(w2b, cfg2, toks), 2 * a)                # the head is the last, linear step
    # positions shifted as a whole change nothing (rotation depends on distance only)
    assert np.allclose(P.forward(w, cfg, toks, start_pos=17), full)


def test_each_half_of_a_layer_has_its_own_norm():
    """One token, one layer: softmax over the single visible key is 1, so the mixer's output is
    W_o applied to the value heads (each repeated for its query heads), and the whole layer can be
    written out by hand.  The two norms get different constant weights a and b: swapping them, or
    using one for both halves, changes the result."""
    rng = np.random.default_rng(21)
    D, F, V, H, G, d = 6, 5, 7, 2, 1, 4
    a, b, c = 0.5, 3.0, 1.25
    cfg = dict(num_hidden_layers=1, num_attention_heads=H, num_key_value_heads=G, head_dim=d, rms_norm_eps=1e-5,
               rope_theta=100.0)
    p = "model.layers.0."
    w = {"model.embed_tokens.weight": rng.standard_normal((V, D)), "model.norm.weight": np.full(D, c),
         p + "input_layernorm.weight": np.full(D, a), p + "post_attention_layernorm.weight": np.full(D, b),
         p + "self_attn.q_proj.weight": rng.standard_normal((H * d, D)),
         p + "self_attn.k_proj.weight": rng.standard_normal((G * d, D)),
         p + "self_attn.v_proj.weight": rng.standard_normal((G * d, D)),
         p + "self_attn.o_proj.weight": rng.standard_normal((D, H * d)),
         p + "mlp.gate_proj.weight": rng.standard_normal((F, D)), p + "mlp.up_proj.weight": rng.standard_normal((F, D)),
         p + "mlp.down_proj.weight": rng.standard_normal((D, F)), "lm_head.weight": rng.standard_normal((V, D))}

    def unit(x):
        return x / math.sqrt(float(x @ x) / D + 1e-5)

    def by_hand(first, second):
        x = w["model.embed_tokens.weight"][3]
        v = w[p + "self_attn.v_proj.weight"] @ (first * unit(x))
        x = x + w[p + "self_attn.o_proj.weight"] @ np.concatenate([v] * (H // G))
        h = second * unit(x)
        g, u = w[p + "mlp.gate_proj.weight"] @ h, w[p + "mlp.up_proj.weight"] @ h
        x = x + w[p + "mlp.down_proj.weight"] @ (g / (1.0 + np.exp(-g)) * u)
        return w["lm_head.weight"] @ (c * unit(x))

    got = P.forward(w, cfg, [3])[0]
    assert np.allclose(got, by_hand(a, b), rtol=1e-12)
    assert not np.allclose(got, by_hand(b, a), rtol=1e-3)
    assert not np.allclose(got, by_hand(a, a), rtol=1e-3) and not np.allclose(got, by_hand(b, b), rtol=1e-3)


# ---------------------------------------------------------------------------------------- sampler
def test_xorshift64_known_value_and_uniform():
    assert SP.xorshift64(1) == 1082269761                    # 1 -> 8193 -> 8257 -> 8257 ^ (8257 << 17)
    assert SP.init_state(0) == 42 and SP.init_state(5) == 5
    # (float)(x >> 11) / (float)(1 << 53), sampler.c:19-21: the 53-bit integer is rounded to the 24
    # bits of a float before the division.  Expected values from exact integer arithmetic: state
    # 42 gives x >> 11 = 22194729, which is odd beyond 2^24 and rounds to 22194728
    r, s = SP.rand_float(42)
    assert s == 45454805674 and s >> 11 == 22194729
    assert r == float.fromhex("0x1.52aa28p-29") == 22194728 / 2.0 ** 53
    r, s = SP.rand_float(0x123456789ABCDEF)
    assert s == 4550888344034083252 and s >> 11 == 2222113449235392
    assert r == float.fromhex("0x1.f94006p-3") == 2222113402388480 / 2.0 ** 53     # not 2222113449235392 / 2^53


def test_sampler_special_cases():
    rng = np.random.default_rng(9)
    logits = rng.standard_normal(50).astype(np.float32)
    top = int(np.argmax(logits))
    assert SP.sample(logits, 0.0, 0, 1.0, 0.0, 42) == (top, 42)          # greedy draws nothing
    tie = np.zeros(5, dtype=np.float32)
    tie[[1, 3]] = 2.0
    assert SP.argmax_first(tie) == 1
    s = 42
    for _ in range(20):
        t1, s1 = SP.sample(logits, 0.8, 1, 1.0, 0.0, s)                  # top_k = 1
        t2, _ = SP.sample(logits, 0.8, 0, 1e-9, 0.0, s)                  # a tiny top_p keeps one
        t3, _ = SP.sample(logits, 0.8, 0, 1.0, 1.0, s)                   # min_p = 1 keeps the maximum only
        t4, _ = SP.sample(logits, 1e-4, 0, 1.0, 0.0, s)                  # T -> 0
        assert t1 == t2 == t3 == t4 == top
        s = s1


def test_sampler_frequencies_follow_softmax_of_logits_over_t():
    logits = np.array([2.0, 1.0, 0.5, 0.0, -1.0, -3.0], dtype=np.float32)
    T = 0.7
    p = np.exp(logits / T) / np.exp(logits / T).sum()
    counts = np.zeros(6)
    s = SP.init_state(123)
    n = 6000
    for _ in range(n):
        t, s = SP.sample(logits, T, 0, 1.0, 0.0, s)
        counts[t] += 1
    chi2 = ((counts - n * p) ** 2 / (n * p)).sum()
    assert chi2 < 25.0                                                   # 5 degrees of freedom: p < 1e-4
    # top_p is measured on the T = 1 distribution, top_k cuts first
    p1 = np.exp(logits) / np.exp(logits).sum()
    keep = int(np.searchsorted(np.cumsum(p1), 0.8) + 1)
    seen = set()
    for _ in range(500):
        t, s = SP.sample(logits, 5.0, 0, 0.8, 0.0, s)
        seen.add(t)
    assert seen == set(range(keep))
