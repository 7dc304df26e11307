"""A model with its cache and workspace: the object that generation and trace replay drive.

`begin` gives each new sequence a slot, `step` runs a batch of them from the cache and
returns logits at the wanted rows, `release` gives slots and pages back.  A step never
runs tokens it was not given: the prompt once, then one token each.

A model whose parts all emit operations of a launch program (`DecoderModel.program`) is stepped
by the engine in the library: the cache's books, the step's index arrays, the workspace and the
recorded decode steps live there, and a step is one call (picolm's model_forward and
model_forward_prefill are such calls too, picolm/model.h:538-539).  A model with a part that
only has a Python `forward` is stepped part by part from here, with the same kernels.
"""
from __future__ import annotations

import gc

import torch

from ..cache import Cache, CacheFull
from ..cache.slots import PAGE_TOKENS
from ..parts.base import Workspace
from .batch import DecodeBatch, StepBatch, StepError, decode_pages_per_chunk
from .model import DecoderModel


class _DecodeGraph:
    """The kernel launches of one decode step of `n_seq` sequences, recorded as a HIP graph."""

    def __init__(self, session: "Session", n_seq: int, pages_per_chunk: int):
        reserve = sum(DecodeBatch.ints_for(n_seq, pages_per_chunk, g.table_host.shape[1]) for g in session.cache.kv)
        self.batch = DecodeBatch(n_seq, pages_per_chunk, session.model.runtime.device, reserve)
        self.workspace = Workspace(session.model.runtime.device)      # its own: recorded addresses must stay
        self.graph = None
        self.logits = None
        self.uses = 0

    def run(self, s: "Session", slots, pos0, tokens, tokens_on_device=None) -> torch.Tensor:
        self.batch.fill(slots, pos0, tokens, s.cache.version, tokens_on_device)
        self.uses += 1
        if self.graph is not None:
            self.graph.replay()
            return self.logits
        logits = s.model.step(s.cache, self.batch, self.workspace)
        if self.uses >= 2:
            # the sizes have been seen, so the workspace is allocated: record the same launches
            # (recording runs nothing; this step's result came from the eager run above)
            # Python's collector must not run while the stream records: freeing a GPU object
            # in the middle of a recording aborts the process
            g = torch.cuda.CUDAGraph()
            was_enabled = gc.isenabled()
            gc.disable()
            try:
                with torch.cuda.graph(g):
                    self.logits = s.model.step(s.cache, self.batch, self.workspace)
            finally:
                if was_enabled:
                    gc.enable()
            self.graph = g
            self.batch.frozen = True
        return logits


class Session:
    def __init__(self, model: DecoderModel, max_tokens: int, max_seq_len: int | None = None,
                 n_slots: int | None = None, graphs: bool = True, native: bool | None = None, time_ops: bool = False):
        """`native`: None steps in the library when the model's parts allow it, False steps from
        Python part by part, True insists on the library.  `time_ops` (library only): GPU time is
        kept by class of operation (`engine.op_times()`), and decode steps are launched one by one."""
        if model.runtime is None:
            raise StepError("the model has no weights loaded")
        self.model = model
        self.vocab_size = model.head.V
        self.engine = None
        if native is not False:
            limit = getattr(model.config, "max_position_embeddings", None) or max_tokens
            seq_len = min(max_seq_len or limit, limit)
            for b in model.blocks:          # tables for every position the cache can hold
                b.mixer.prepare(model.runtime, min(seq_len, (max_tokens + PAGE_TOKENS - 1) // PAGE_TOKENS * PAGE_TOKENS))
            built = model.program()
            if built is not None:
                from .native import EngineCache, NativeEngine
                self.engine = NativeEngine(built, max_tokens, seq_len, n_slots, model.runtime.device, graphs=graphs, time_ops=time_ops)
                self.cache = EngineCache(self.engine, model.cache_spec, model.runtime.dtype, model.runtime.device)
                self.graphs = graphs
                return
            if native:
                raise StepError("a part of this model has no operations of the engine's; it is stepped from Python")
        self.cache: Cache = model.new_cache(max_tokens, max_seq_len, n_slots)
        self.workspace = Workspace(model.runtime.device)
        # decode steps replay recorded HIP graphs when every part's launches depend on device
        # memory only (a part says so with `graph_safe`)
        self.graphs = graphs and model.graph_safe()
        self._decode_graphs: dict[tuple, _DecodeGraph] = {}
        self._decode_geometry: dict[int, tuple] = {}

    # -- slots -------------------------------------------------------------------------------
    def begin(self, n: int = 1) -> list[int]:
        """Slots for `n` new sequences; on failure none is kept."""
        alloc = self.engine.slot_alloc if self.engine is not None else self.cache.alloc_slot
        got = []
        try:
            for _ in range(n):
                got.append(alloc())
        except CacheFull:
            self.release(got)
            raise
        return got

    def release(self, slots) -> None:
        free = self.engine.slot_free if self.engine is not None else self.cache.free_slot
        for s in slots:
            free(s)

    def recorded_steps(self) -> int:
        """Decode steps (by batch size and chunking) that replay a recorded HIP graph."""
        if self.engine is not None:
            return self.engine.recorded_steps()
        return sum(g.graph is not None for g in self._decode_graphs.values())

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    # -- the step ------------------------------------------------------------------------------
    def step(self, slots, new_tokens, want=None) -> torch.Tensor:
        """Run `new_tokens[i]` for the sequence in `slots[i]`, appended at its current
        length.  `want[i]` lists indices into new_tokens[i]; default: each sequence's last
        token.  Returns float32 logits [sum(len(want[i])), vocab] in the order of the
        sequences and of `want`; the tensor is workspace memory, valid until the next step.
        """
        slots = list(slots)
        if self.engine is not None:
            return self.engine.step(slots, new_tokens, want)
        for s in slots:
            if not self.cache.slots.is_live(s):
                raise StepError(f"slot {s} is not live")
        if want is None:
            want = [[len(t) - 1] for t in new_tokens]
        pos0 = [self.cache.length(s) for s in slots]
        n_new = [len(t) for t in new_tokens]
        if self.graphs and slots and max(n_new) == 1 and min(n_new) == 1 and all(list(w) == [0] for w in want):
            return self._decode_step(slots, pos0, [int(t[0]) for t in new_tokens])
        batch = StepBatch(slots, pos0, new_tokens, want, self.vocab_size, self.model.runtime.device)
        self.cache.reserve_many(slots, [p + n for p, n in zip(pos0, n_new)])
        self.cache.flush()
        logits = self.model.step(self.cache, batch, self.workspace)
        for s, p, n in zip(slots, pos0, n_new):
            self.cache.set_length(s, p + n)
        return logits

    def step_tokens_on_device(self, slots, tokens: torch.Tensor) -> torch.Tensor:
        """One more token for each sequence, the tokens being an int32 tensor on the device that
        the host need not have seen: what a sampling kernel wrote, or will have written when the
        step runs.  Nothing here waits for the GPU, so the step can be handed over while the one
        that produces its tokens still runs.  The tokens must lie inside the vocabulary (a
        sampler's do); logits as from `step`, one row a sequence."""
        slots = list(slots)
        device = torch.device(self.model.runtime.device)
        if tokens.dtype != torch.int32 or tokens.shape != (len(slots),) or tokens.device.type != device.type:
            raise StepError(f"tokens on the device: expected int32 [{len(slots)}] on {device}, "
                            f"got {tokens.dtype} {tuple(tokens.shape)} on {tokens.device}")
        if self.engine is not None:
            return self.engine.step_device_tokens(slots, tokens.contiguous())
        for s in slots:
            if not self.cache.slots.is_live(s):
                raise StepError(f"slot {s} is not live")
        if not (self.graphs and slots):
            return self.step(slots, [[t] for t in tokens.tolist()])
        return self._decode_step(slots, [self.cache.length(s) for s in slots], None, tokens)

    def _decode_step(self, slots, pos0, tokens, tokens_on_device=None) -> torch.Tensor:
        if len(set(slots)) != len(slots):
            raise StepError("a slot appears twice in one step")
        for t in tokens or ():
            if not 0 <= t < self.vocab_size:
                raise StepError(f"token id {t} is outside the vocabulary of {self.vocab_size}")
        # unless a sequence starts a page (or runs out of room), its new token stays in its last page
        grow = [(s, p + 1) for s, p in zip(slots, pos0) if p % PAGE_TOKENS == 0 or p >= self.cache.max_seq_len]
        if grow:
            self.cache.reserve_many([s for s, _ in grow], [n for _, n in grow])
            self.cache.flush()
        geometry = self._decode_geometry.get(len(slots))
        if geometry is None:
            geometry = self._decode_geometry[len(slots)] = self.model.decode_geometry(len(slots))
        ppc = decode_pages_per_chunk(pos0, *geometry)
        key = (len(slots), ppc)
        g = self._decode_graphs.get(key)
        if g is None:
            g = self._decode_graphs[key] = _DecodeGraph(self, len(slots), ppc)
        logits = g.run(self, slots, pos0, tokens, tokens_on_device)
        for s, p in zip(slots, pos0):
            self.cache.set_length(s, p + 1)
        return logits
