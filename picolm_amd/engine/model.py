"""A decoder put together from parts, and its launch program.

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
from ..cache import CacheSpec, KVGroupSpec, StateGroupSpec
from ..parts.base import CacheBinding, Runtime, Workspace
from ..weights import WeightFetcher, check_specs
from .errors import StepError


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

    def prepare(self, max_positions: int) -> None:
        """Let the mixers lay out what depends on the longest sequence (rotary tables)."""
        for b in self.blocks:
            b.mixer.prepare(self.runtime, max_positions)

    # -- the model as a launch program --------------------------------------------------------
    def program(self):
        """The model as the flat list of operations that the engine in the library walks
        (engine/program.py): embedding -> the layer calls of `order` -> final norm on the wanted
        rows -> head.  Every part emits what it is: operations of the engine's own, or a call of its
        `forward`.  The mixers must have been prepared (`prepare`) for the positions the engine
        will see."""
        from .program import ROWS_WANTED, ProgramBuilder
        from ..parts.block import norm_ref_of
        if self.runtime is None:
            raise StepError("the model has no weights loaded")
        ws = Workspace(self.runtime.device)
        for part in self.parts():
            part.bind_runtime(self.runtime, ws)
        b = ProgramBuilder(self.runtime.dtype)
        x = self.embedding.emit(b)
        for i, (call, binding) in enumerate(zip(self.order, self.bindings)):
            b.binding = binding
            # a block is told which norm meets the residual stream after it (the next block's first
            # one, or the final norm when every row's logits are wanted), so that its last product
            # can prepare that norm
            if i + 1 < len(self.order):
                nxt = self.blocks[self.order[i + 1].block].first_norm()
                self.blocks[call.block].emit(b, x, norm_ref_of(nxt) if nxt is not None else None, 0)
            else:
                self.blocks[call.block].emit(b, x, norm_ref_of(self.final_norm), 1)
        b.binding = None
        self.head.emit(b, self.final_norm.emit(b, x, ROWS_WANTED))
        return b.finish(self.head.V, self.cache_spec)
