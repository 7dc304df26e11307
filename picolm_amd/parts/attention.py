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

from .. import kernels
from ..cache.kv import WINDOW_STEP_TOKENS
from .base import KVRequest, Mixer, Runtime, StepContext
from .linear import Linear
from .position import NoPosition, PositionEncoding
import torch


MAX_HEAD_DIM = 256      # what a tile of the vector-ALU attention kernel holds in LDS


class Attention(Mixer):
    graph_safe = True      # launches depend on device memory only
    takes_normed_rows = True   # the input goes to a Linear unchanged

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

    def decode_geometry(self, dtype, n_seq: int):
        """(workgroups per chunk, most pages a chunk should have) of this layer's decode
        attention: what sizes the step's work list."""
        return kernels.attn_decode_geometry(dtype, n_seq, self.H, self.G, self.d)

    def prepare(self, runtime: Runtime, max_positions: int) -> None:
        self.position.prepare(runtime, max_positions)

    def emit(self, b, norm, x: int, out_norm=None, out_norm_when: int = 0) -> None:
        """x += o(attention(rotate(q, k), v)) with q, k, v = W norm(x), as operations of a launch
        program.  The engine runs rotations (or no position encoding) and keeps all keys."""
        from ..engine.program import CannotEmit
        from .position import RotaryEmbedding
        if type(self) is not Attention or type(self.position) not in (RotaryEmbedding, NoPosition):
            raise CannotEmit("an attention or position encoding of another kind than the engine runs")
        if self.window:
            raise CannotEmit("the engine keeps all keys; a window of them is stepped from Python")
        H, G, d = self.H, self.G, self.d
        h = b.buffer("norm.out", self.qkv.in_size, b.dtype)
        qkv = b.buffer("attn.qkv", (H + 2 * G) * d, torch.float32)
        self.qkv.emit(b, h, qkv, kernels.EPI_STORE, in_norm=norm, in_norm_x=x)
        q = b.buffer("attn.q", H * d, b.dtype)
        out = b.buffer("attn.out", H * d, b.dtype)
        b.attention(qkv, q, out, H, G, d, self.window, self.scale, self.position.rotary_tables())
        self.o.emit(b, out, x, kernels.EPI_ACCUMULATE, out_norm=out_norm, out_norm_when=out_norm_when)

    def forward(self, ctx: StepContext, h, residual) -> None:
        b = ctx.batch
        H, G, d = self.H, self.G, self.d
        T = h.shape[0]
        qkv = ctx.ws.get("attn.qkv", (T, (H + 2 * G) * d), torch.float32)
        self.qkv.forward(h, qkv)
        k_pages, v_pages, table, ring = ctx.kv()
        tables = self.position.rotary_tables()
        if tables is None:
            self.position.apply(ctx, qkv, H, G, d)
            cos = sin = None
            style = 0
        else:
            cos, sin, style = tables
        q = ctx.ws.get("attn.q", (T, H * d), ctx.dtype)
        out = ctx.ws.get("attn.out", (T, H * d), ctx.dtype)
        writes = ctx.binding.writes
        kp, vp = (k_pages, v_pages) if writes else (None, None)
        group, table_host = ctx.kv_host()
        tok_page = b.write_pages(group, table_host, ring) if writes else None
        if b.is_decode:
            chunk_list, n_chunks, ppc, most = b.decode_chunks(*self.decode_geometry(ctx.dtype, b.n_seq), self.window,
                                                               group, table_host, ring)
            partial = ctx.ws.get("attn.partial", (b.n_seq * H * most * (d + 2),), torch.float32) if most > 1 else None
            done = ctx.ws.zeros("attn.chunks_done", (kernels.attn_decode_counters(b.n_seq, H, G),), torch.int32) if most > 1 else None
            if writes and kernels.attn_decode_rope_takes(ctx.dtype, d):
                # rotation (if the position encoding is one), cache write and attention in one launch
                kernels.attn_decode_rope(qkv, k_pages, v_pages, out, partial, b.n_seq, chunk_list, n_chunks, ppc, most,
                                         b.seq_pos0, table, ring, H, G, d, self.window, self.scale, cos, sin, style,
                                         tok_page, done)
            else:
                kernels.rope_kv_store(qkv, q, kp, vp, cos, sin, style, b.tok_pos, tok_page, H, G, d)
                kernels.attn_decode(q, k_pages, v_pages, out, partial, b.n_seq, chunk_list, n_chunks, ppc, most,
                                    b.seq_pos0, table, ring, H, G, d, self.window, self.scale, done)
        elif self.window > 0 and ring < table.shape[1] and b.max_new > WINDOW_STEP_TOKENS:
            # a ring holds a window and one chunk: write and answer the step chunk by chunk
            for c in b.chunks(WINDOW_STEP_TOKENS):
                kernels.rope_kv_store(qkv, q, kp, vp, cos, sin, style, b.tok_pos, tok_page, H, G, d,
                                      rows=c.rows, n_rows=c.n_rows)
                kernels.attn_prefill(q, k_pages, v_pages, out, c, table, ring, H, G, d, self.window, self.scale)
        elif kernels.attn_prefill_rope_takes(ctx.dtype, d, T):
            # keys and values go to the cache; the attention kernel rotates q on its way in
            if writes:
                kernels.kv_store_tiles(qkv, kp, vp, cos, sin, style, b, table, ring, H, G, d)
            kernels.attn_prefill_rope(qkv, k_pages, v_pages, out, b, table, ring, H, G, d, self.window, self.scale, cos, sin, style)
        else:
            kernels.rope_kv_store(qkv, q, kp, vp, cos, sin, style, b.tok_pos, tok_page, H, G, d)
            kernels.attn_prefill(q, k_pages, v_pages, out, b, table, ring, H, G, d, self.window, self.scale)
        self.o.forward(out, residual, kernels.EPI_ACCUMULATE, ctx)
