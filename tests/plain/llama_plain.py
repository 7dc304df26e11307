"""Plain, slow Llama decoder in NumPy float64: whole sequences, no cache, one function a part.

Written from the formulas of whoreson/picolm (cited as file:line of its picolm/ folder).
It shares no code with picolm_amd: tests compare the engine against it.
The llama3 frequency scaling is not in the reference; its definition here follows the
parameter names of the model's config.json (`rope_scaling`).
"""
from __future__ import annotations

import math

import numpy as np

F64 = np.float64


# ----------------------------------------------------------------------------- position encoding
def rope_inv_freq(head_dim: int, theta: float, scaling: dict | None = None) -> np.ndarray:
    """Inverse frequencies f_i = base^(-2i/d), i in [0, d/2).

    model_core.c:321 computes `theta = pos / powf(base, 2i/rope_dim)`; the inverse
    frequency is the factor of `pos` in it.  With `scaling` (rope_type "llama3") long
    wavelengths are divided by `factor`, short ones kept, the band between blended
    linearly in the ratio original_max/wavelength.
    """
    i = np.arange(head_dim // 2, dtype=F64)
    inv = 1.0 / np.power(F64(theta), 2.0 * i / F64(head_dim))
    if scaling is None:
        return inv
    factor = F64(scaling["factor"])
    low = F64(scaling["low_freq_factor"])
    high = F64(scaling["high_freq_factor"])
    orig = F64(scaling["original_max_position_embeddings"])
    out = np.empty_like(inv)
    for j, f in enumerate(inv):
        wavelen = 2.0 * math.pi / f
        if wavelen < orig / high:
            out[j] = f
        elif wavelen > orig / low:
            out[j] = f / factor
        else:
            s = (orig / wavelen - low) / (high - low)
            out[j] = (1.0 - s) * f / factor + s * f
    return out


def rope_tables(positions: np.ndarray, inv_freq: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """cos/sin of pos * f_i, [n_pos, d/2] (model_core.c:317-324)."""
    ang = np.asarray(positions, dtype=F64)[:, None] * inv_freq[None, :]
    return np.cos(ang), np.sin(ang)


def apply_rope(x: np.ndarray, cos: np.ndarray, sin: np.ndarray, style: str) -> np.ndarray:
    """Rotate x[T, n_heads, d] by its position's angles.

    pairwise: (x[2i], x[2i+1]) <- (x0*c - x1*s, x0*s + x1*c)   tensor.c:3298-3302
    half:     (x[i], x[i+d/2]) the same way                     tensor.c:3219-3228
    """
    out = np.array(x, dtype=F64, copy=True)
    c = cos[:, None, :]
    s = sin[:, None, :]
    if style == "pairwise":
        x0, x1 = x[..., 0::2], x[..., 1::2]
        out[..., 0::2] = x0 * c - x1 * s
        out[..., 1::2] = x0 * s + x1 * c
    elif style == "half":
        half = x.shape[-1] // 2
        x0, x1 = x[..., :half], x[..., half:]
        out[..., :half] = x0 * c - x1 * s
        out[..., half:] = x0 * s + x1 * c
    else:
        raise ValueError(style)
    return out


# ----------------------------------------------------------------------------- norm
def rmsnorm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """out_i = (x_i * r) * w_i with r = 1/sqrt(sum(x^2)/size + eps)  (tensor.c:2942, :3001, :3062)."""
    x = np.asarray(x, dtype=F64)
    ss = np.sum(x * x, axis=-1, keepdims=True)
    r = 1.0 / np.sqrt(ss / x.shape[-1] + eps)
    return (x * r) * np.asarray(weight, dtype=F64)


# ----------------------------------------------------------------------------- mixer
def softmax_rows(s: np.ndarray) -> np.ndarray:
    """Row softmax with the maximum subtracted first (tensor.c:3066-3076)."""
    m = np.max(s, axis=-1, keepdims=True)
    e = np.exp(s - m)
    return e / np.sum(e, axis=-1, keepdims=True)


def causal_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, window: int = 0) -> np.ndarray:
    """q[T,H,d], k/v[T,G,d] -> [T,H,d].

    Query head h reads KV head h // (H/G); score = (q.k) * 1/sqrt(d); key t is visible
    to query p iff t <= p (model_attention.c:54, :70; scale model_core.c:2077), and with
    a window w > 0 only iff p - t < w.  softmax then the weighted sum of V
    (model_attention.c:72-123, written there as an online recurrence).
    """
    T, H, d = q.shape
    G = k.shape[1]
    rep = H // G
    scale = 1.0 / math.sqrt(d)
    out = np.zeros((T, H, d), dtype=F64)
    pos = np.arange(T)
    visible = pos[None, :] <= pos[:, None]
    if window > 0:
        visible &= (pos[:, None] - pos[None, :]) < window
    for h in range(H):
        g = h // rep
        s = (q[:, h, :] @ k[:, g, :].T) * scale
        s = np.where(visible, s, -np.inf)
        out[:, h, :] = softmax_rows(s) @ v[:, g, :]
    return out


def attention_block(x, w, prefix, cfg, positions):
    """q,k,v = W x (no bias; model_core.c:1849,:1877,:1975); rope on q and k before the cache
    (:1908); attention; o-projection (:2149)."""
    H, G, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    T = x.shape[0]
    q = (x @ w[prefix + "q_proj.weight"].T).reshape(T, H, d)
    k = (x @ w[prefix + "k_proj.weight"].T).reshape(T, G, d)
    v = (x @ w[prefix + "v_proj.weight"].T).reshape(T, G, d)
    inv = rope_inv_freq(d, cfg["rope_theta"], cfg.get("rope_scaling"))
    cos, sin = rope_tables(positions, inv)
    q = apply_rope(q, cos, sin, cfg.get("rope_style", "pairwise"))
    k = apply_rope(k, cos, sin, cfg.get("rope_style", "pairwise"))
    a = causal_attention(q, k, v, cfg.get("window", 0)).reshape(T, H * d)
    return a @ w[prefix + "o_proj.weight"].T


# ----------------------------------------------------------------------------- feed-forward
def silu(x: np.ndarray) -> np.ndarray:
    """x / (1 + exp(-x))  (tensor.c:3306-3315)."""
    return x / (1.0 + np.exp(-x))


def swiglu(x, w_gate, w_up, w_down):
    """down(silu(gate x) * (up x))  (model_core.c:2182-2199)."""
    return (silu(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


# ----------------------------------------------------------------------------- whole model
def as_f64(weights: dict) -> dict:
    return {k: np.asarray(v, dtype=F64) for k, v in weights.items()}


def forward(weights: dict, cfg: dict, tokens, start_pos: int = 0) -> np.ndarray:
    """Logits [T, V] of one whole sequence.

    embed (model_core.c:1785) -> per layer: x += attn(rmsnorm(x)); x += ffn(rmsnorm(x))
    (:1841, :2151, :2160, :2204) -> final rmsnorm (:2213) -> head (:2220); the head is the
    embedding table when lm_head.weight is absent (safetensors.c:248-251).
    """
    w = weights
    tokens = np.asarray(tokens, dtype=np.int64)
    positions = np.arange(start_pos, start_pos + len(tokens))
    eps = cfg["rms_norm_eps"]
    x = w["model.embed_tokens.weight"][tokens]
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        h = rmsnorm(x, w[p + "input_layernorm.weight"], eps)
        x = x + attention_block(h, w, p + "self_attn.", cfg, positions)
        h = rmsnorm(x, w[p + "post_attention_layernorm.weight"], eps)
        x = x + swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                       w[p + "mlp.down_proj.weight"])
    x = rmsnorm(x, w["model.norm.weight"], eps)
    head = w.get("lm_head.weight", w["model.embed_tokens.weight"])
    return x @ head.T
