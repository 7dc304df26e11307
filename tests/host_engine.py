"""An engine of the library's without a GPU (the host-only flag): it keeps slots, pages and page
tables and plans every step's index arrays, holds no device memory and launches nothing.  The
program has made-up weights that nothing reads."""
import ctypes

import torch

from picolm_amd.cache import CacheSpec, KVGroupSpec, StateGroupSpec
from picolm_amd.engine import program as P
from picolm_amd.engine.native import NativeEngine
from picolm_amd.parts.base import CacheBinding

D, H, G, d, V = 64, 4, 2, 16, 100


def host_engine(max_tokens=64 * 10, max_seq_len=64 * 4, n_slots=3, layers=2, windows=(0,), v_head_dim=0, state_shape=None):
    """`layers` attention layers and a head; layer l keeps keys and values in the group of
    windows[l % len(windows)] (0: all keys).  state_shape: also a called operation per layer with a
    state entry of that shape."""
    b = P.ProgramBuilder(torch.float32, host_only=True)
    x = b.buffer("residual", D, torch.float32)
    b.embed(torch.zeros(V, D), x)
    norm = P.NormRef(torch.ones(D), 1e-5)
    counts = [0] * len(windows)
    nothing = P.CALL_FN(lambda user, view: 0)
    for layer in range(layers):
        g = layer % len(windows)
        b.binding = CacheBinding((g, counts[g]), (0, layer) if state_shape else None, True)
        counts[g] += 1
        h = b.buffer("norm.out", D, torch.float32)
        qkv = b.buffer("attn.qkv", (H + 2 * G) * d, torch.float32)
        b.linear(torch.zeros((H + 2 * G) * d, D), P.Rows(h, norm, x), qkv, 0)
        q, o = b.buffer("attn.q", H * d, torch.float32), b.buffer("attn.out", H * d, torch.float32)
        if v_head_dim:
            b.call(nothing, out=o, inp=qkv, uses_kv=True, attends=True, tile_rows=16)
        else:
            b.attention(qkv, q, o, H, G, d, windows[g], 0.25, None)
        if state_shape:
            b.call(nothing, out=x, uses_state=True)
        b.linear(torch.zeros(D, H * d), o, x, 1, out_norm=norm, out_norm_when=int(layer == layers - 1))
    hf = b.buffer("norm.final", D, torch.float32, P.ROWS_WANTED)
    lg = b.buffer("logits", V, torch.float32, P.ROWS_WANTED)
    b.linear(torch.zeros(V, D), P.Rows(hf, norm, x), lg, 0, rows=P.ROWS_WANTED)
    b.logits_buffer = lg
    spec = CacheSpec([KVGroupSpec(n, G, d, w, v_head_dim) for w, n in zip(windows, counts) if n],
                     [StateGroupSpec(layers, tuple(state_shape))] if state_shape else [])
    return NativeEngine(b.finish(V, spec), max_tokens, max_seq_len, n_slots, "cpu", host_only=True)
