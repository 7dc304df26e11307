"""A decoder put together from parts, and its one step function.

embedding -> the layer calls of `order` -> final norm on the wanted rows -> head
(picolm/model_core.c:1785, :1799-2210, :2213, :2220).  `order` is data: a list of layer
calls, each naming a block (a block may be named twice) and either owning a cache entry or
reading the entry of an earlier call.  Cache groups are derived from what the mixers ask
for: calls whose mixers need the same kind of keys and values (heads, head size, window)
share a group and its storage, as picolm's kv_layer_map does for its one kind
(picolm/model_core.c:668-681).
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import kernels
from ..cache import Cache, CacheSpec, KVGroupSpec, StateGroupSpec
from ..parts.base import CacheBinding, Runtime, StepContext, Workspace
from ..weights import WeightFetcher, check_specs
from .batch import StepBatch, StepError


@dataclass(frozen=True)
class LayerCall:
    block: int                          # index into the model's blocks
    reads_cache_of: int | None = None   # index of an earlier call whose cache entry this one reads


class DecoderModel:
    def __init__(self, config, embedding, blocks, final_norm, head, order=None):
        self.config = config
        self.embedding = embedding
        self.blocks = list(blocks)
        self.final_norm = final_norm
        self.head = head
        order = list(range(len(self.blocks))) if order is None else list(order)
        self.order = [c if isinstance(c, LayerCall) else LayerCall(int(c)) for c in order]
        for i, c in enumerate(self.order):
            if not 0 <= c.block < len(self.blocks):
                raise ValueError(f"layer call {i} names block {c.block}, there are {len(self.blocks)}")
            if c.reads_cache_of is not None and not 0 <= c.reads_cache_of < i:
                raise ValueError(f"layer call {i} can only read the cache of an earlier call")
        self.runtime: Runtime | None = None
        self._plan_cache()

    # -- structure --------------------------------------------------------------------------
    def parts(self):
        return [self.embedding, *self.blocks, self.final_norm, self.head]

    def tensor_specs(self):
        out, seen = [], set()
        for p in self.parts():
            for s in p.all_specs():
                if s.name not in seen:
                    seen.add(s.name)
                    out.append(s)
        return out

    def _plan_cache(self) -> None:
        kv_keys, state_keys = [], []
        kv_counts, state_counts = [], []
        self.bindings: list[CacheBinding] = []
        for i, call in enumerate(self.order):
            kv_req, st_req = self.blocks[call.block].mixer.cache_requests()
            if call.reads_cache_of is not None:
                src = self.bindings[call.reads_cache_of]
                src_call = self.order[call.reads_cache_of]
                if self.blocks[src_call.block].mixer.cache_requests() != (kv_req, st_req):
                    raise ValueError(f"layer call {i} reads a cache of another shape than it needs")
                self.bindings.append(CacheBinding(src.kv, src.state, writes=False))
                continue
            kv = st = None
            if kv_req is not None:
                if kv_req not in kv_keys:
                    kv_keys.append(kv_req)
                    kv_counts.append(0)
                g = kv_keys.index(kv_req)
                kv = (g, kv_counts[g])
                kv_counts[g] += 1
            if st_req is not None:
                if st_req not in state_keys:
                    state_keys.append(st_req)
                    state_counts.append(0)
                g = state_keys.index(st_req)
                st = (g, state_counts[g])
                state_counts[g] += 1
            self.bindings.append(CacheBinding(kv, st, writes=True))
        self.cache_spec = CacheSpec(
            [KVGroupSpec(n, k.n_kv_heads, k.head_dim, k.window, k.v_head_dim) for k, n in zip(kv_keys, kv_counts)],
            [StateGroupSpec(n, tuple(k.shape), k.dtype) for k, n in zip(state_keys, state_counts)])

    def graph_safe(self) -> bool:
        """Whether a decode step's launches depend on device memory only, so that they can be
        recorded once and replayed."""
        def safe(p):
            return getattr(p, "graph_safe", False) and all(safe(c) for c in p.children())
        return all(safe(p) for p in self.parts())

    def decode_geometry(self, n_seq: int) -> tuple[int, int]:
        """(workgroups per chunk, most pages a chunk should have) over the mixers that run a
        decode attention: the widest launch and the tightest limit size the step's work list."""
        per_chunk, max_pages = 1, 64
        for b in self.blocks:
            f = getattr(b.mixer, "decode_geometry", None)
            if f is not None:
                p, m = f(self.runtime.dtype, n_seq)
                per_chunk, max_pages = max(per_chunk, p), min(max_pages, m)
        return per_chunk, max_pages

    # -- weights ----------------------------------------------------------------------------
    def load(self, source, runtime: Runtime) -> "DecoderModel":
        """Check `source` against every declared tensor, then bind."""
        kernels.require_device()
        check_specs(source, self.tensor_specs())
        self.runtime = runtime
        fetch = WeightFetcher(source, runtime.device, runtime.dtype)
        for p in self.parts():
            p.load_all(fetch, runtime)
        return self

    def weight_bytes(self) -> int:
        """Bytes of the declared tensors at the runtime's element size: about what a decode step reads."""
        size = self.runtime.dtype.itemsize if self.runtime is not None else 2
        total = 0
        for spec in self.tensor_specs():
            n = 1
            for d in spec.shape:
                n *= int(d)
            total += n * size
        return total

    def new_cache(self, max_tokens: int, max_seq_len: int | None = None, n_slots: int | None = None) -> Cache:
        limit = getattr(self.config, "max_position_embeddings", None) or max_tokens
        max_seq_len = min(max_seq_len or limit, limit)
        cache = Cache(self.cache_spec, max_tokens, max_seq_len, self.runtime.dtype, self.runtime.device, n_slots)
        for b in self.blocks:
            b.mixer.prepare(self.runtime, cache.max_seq_len)
        return cache

    # -- the model as a launch program --------------------------------------------------------
    def program(self):
        """The model as the flat list of operations that the engine in the library walks
        (engine/program.py), or None when a part has no such operations: then `step` below runs
        it part by part.  The mixers must have been prepared (`new_cache` does that) for the
        positions the engine will see."""
        from .program import CannotEmit, ProgramBuilder
        if self.runtime is None:
            raise StepError("the model has no weights loaded")
        b = ProgramBuilder(self.runtime.dtype)
        try:
            for part in (self.embedding, self.head, *self.blocks):
                if not callable(getattr(part, "emit", None)):
                    raise CannotEmit(f"{type(part).__name__} has no operations of the engine's")
            final = self.final_norm.norm_ref() if hasattr(self.final_norm, "norm_ref") else None
            if final is None:
                raise CannotEmit(f"{type(self.final_norm).__name__} has no operations of the engine's")
            x = self.embedding.emit(b)
            for i, (call, binding) in enumerate(zip(self.order, self.bindings)):
                b.binding = binding
                if i + 1 < len(self.order):
                    nxt = getattr(self.blocks[self.order[i + 1].block], "first_norm", lambda: None)()
                    after = nxt.norm_ref() if nxt is not None and hasattr(nxt, "norm_ref") else None
                    self.blocks[call.block].emit(b, x, after, 0)
                else:       # the final norm meets every row only in steps that want every row's logits
                    self.blocks[call.block].emit(b, x, final, 1)
            b.binding = None
            self.head.emit(b, final, x)
        except CannotEmit:
            return None
        return b.finish(self.head.V, self.cache_spec)

    # -- the step ---------------------------------------------------------------------------
    def step(self, cache: Cache, batch: StepBatch, workspace: Workspace) -> torch.Tensor:
        """Run the batch's new tokens from the cache; logits [n_want, vocab] float32, a view
        of workspace memory valid until the next step."""
        ctx = StepContext(self.runtime, batch, cache, workspace)
        x = self.embedding.forward(ctx, batch.tokens, batch.T)
        # a block is told which norm meets the residual stream after it (the next block's first one,
        # or the final norm when every row's logits are wanted), so that its last product can
        # prepare that norm (see NormedRows)
        every_row = getattr(batch, "wants_every_row", False)
        for i, (call, binding) in enumerate(zip(self.order, self.bindings)):
            ctx.binding = binding
            block = self.blocks[call.block]
            if i + 1 < len(self.order):
                after = getattr(self.blocks[self.order[i + 1].block], "first_norm", lambda: None)()
            else:
                after = self.final_norm if every_row and batch.n_want else None
            ctx.norm_after_block = after
            block.forward(ctx, x)
        if batch.n_want == 0:
            return workspace.get("logits", (0, self.head.V), torch.float32)
        if every_row:
            h = ctx.normed(self.final_norm, x, self.head)
        else:
            ctx.prepared_norm = None
            h = self.final_norm.forward(ctx, x, rows=batch.want_rows, n_rows=batch.n_want, out_name="norm.final")
        return self.head.forward(ctx, h)
