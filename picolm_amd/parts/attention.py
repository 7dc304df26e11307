"""Causal attention over the cache with grouped KV heads, an optional window, and any
position encoding.

picolm's order (picolm/model_core.c:1849-2151): q, k, v = W x (no bias); rotate q and k;
write k, v to the cache; per query head h, KV head h // (H/G), online softmax of
(q.k)/sqrt(d) over keys t <= pos (picolm/model_attention.c:43-140); output projection; add
into the residual.  q, k and v come from one product over the stacked weights; the
projection back adds into the residual inside the product's epilogue.
"""
from __future__ import annotations

import math

import torch

from .. import kernels
from .base import KVRequest, Mixer, Runtime, forward_is_graph_safe, on_stream, rows_view
from .linear import Linear
from .position import NoPosition, PositionEncoding

MAX_HEAD_DIM = 1024      # what a tile of the vector-ALU attention kernel holds in LDS


class Attention(Mixer):
    graph_safe = True      # launches depend on device memory only

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int,
                 position: PositionEncoding | None = None, window: int = 0, scale: float | None = None,
                 names=("q_proj.weight", "k_proj.weight", "v_proj.weight", "o_proj.weight")):
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} heads do not split over {n_kv_heads} KV heads")
        if not 1 <= head_dim <= MAX_HEAD_DIM:
            raise ValueError(f"head size {head_dim}: the attention kernels take 1 to {MAX_HEAD_DIM}")
        self.H, self.G, self.d = n_heads, n_kv_heads, head_dim
        self.window = int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)   # model_core.c:2077
        self.position = position or NoPosition()
        self.qkv = Linear([prefix + n for n in names[:3]],
                          [n_heads * head_dim, n_kv_heads * head_dim, n_kv_heads * head_dim], hidden_size)
        self.o = Linear([prefix + names[3]], [hidden_size], n_heads * head_dim)

    def children(self):
        return [self.qkv, self.o, self.position]

    def cache_requests(self):
        return KVRequest(self.G, self.d, self.window), None

    def prepare(self, runtime: Runtime, max_positions: int) -> None:
        self.position.prepare(runtime, max_positions)

    def emit(self, b, src, x: int, out_norm=None, out_norm_when: int = 0) -> None:
        """x += o(attention(encode(q, k), v)) with q, k, v = W h for the rows h of `src`, as operations
        of a launch program.  A rotation runs inside the attention operation; a position encoding
        of another kind runs as a call of its `apply` on the float rows of q, k, v before it."""
        H, G, d = self.H, self.G, self.d
        qkv = b.buffer("attn.qkv", (H + 2 * G) * d, torch.float32)
        self.qkv.emit(b, src, qkv, kernels.EPI_STORE)
        tables = self.position.rotary_tables()
        if tables is None and type(self.position).apply is not PositionEncoding.apply:
            position = self.position

            def encode(view):
                with on_stream(view):
                    ctx = position._context(view)
                    position.apply(ctx, rows_view(view.out, view.n_tokens, view.out_row_bytes, torch.float32, ctx.runtime.device),
                                   H, G, d)
            b.call(encode, out=qkv, recordable=forward_is_graph_safe(position, "apply"))
        q = b.buffer("attn.q", H * d, b.dtype)
        out = b.buffer("attn.out", H * d, b.dtype)
        b.attention(qkv, q, out, H, G, d, self.window, self.scale, tables)
        self.o.emit(b, out, x, kernels.EPI_ACCUMULATE, out_norm=out_norm, out_norm_when=out_norm_when)
