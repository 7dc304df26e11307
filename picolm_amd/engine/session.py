"""A model with its cache and workspace: the object that generation and trace replay drive.

`begin` gives each new sequence a slot, `step` runs a batch of them from the cache and
returns logits at the wanted rows, `release` gives slots and pages back.  A step never
runs tokens it was not given: the prompt once, then one token each.

Every model is stepped by the engine in the library (csrc/engine.h), which walks the program that
the model's parts emitted: the cache's books, the step's index arrays, the workspace and the
recorded decode steps live there, and a step is one call (picolm's model_forward and
model_forward_prefill are such calls too, picolm/model.h:538-539).
"""
from __future__ import annotations

import torch

from ..cache import PAGE_TOKENS
from .errors import StepError
from .model import DecoderModel
from .native import EngineCache, NativeEngine


class Session:
    def __init__(self, model: DecoderModel, max_tokens: int, max_seq_len: int | None = None,
                 n_slots: int | None = None, graphs: bool = True, time_ops: bool = False):
        """`max_tokens`: the most tokens live sequences hold together, each sequence's count rounded
        up to pages of 64; `max_seq_len`: the longest one sequence may get (default: the
        configuration's).  `graphs`: decode steps are recorded once and replayed, where every part
        of the model allows it.  `time_ops`: GPU time is kept by class of operation
        (`engine.op_times()`), and decode steps are launched one by one."""
        if model.runtime is None:
            raise StepError("the model has no weights loaded")
        self.model = model
        self.vocab_size = model.head.V
        limit = getattr(model.config, "max_position_embeddings", None) or max_tokens
        seq_len = min(max_seq_len or limit, limit)
        # tables for every position the cache can hold
        model.prepare(min(seq_len, (max_tokens + PAGE_TOKENS - 1) // PAGE_TOKENS * PAGE_TOKENS))
        self.engine = NativeEngine(model.program(), max_tokens, seq_len, n_slots, model.runtime.device, graphs=graphs,
                                   time_ops=time_ops)
        self.cache = EngineCache(self.engine, model.cache_spec, model.runtime.dtype, model.runtime.device)
        self.graphs = graphs and self.engine.program.recordable
        # the most tokens a sequence may bring in one step (0: any number): a called operation on a
        # group with a window sees a step whole, and the group's ring takes in 256 tokens at once
        self.most_new_tokens = self.engine.info(8)

    # -- slots -------------------------------------------------------------------------------
    def begin(self, n: int = 1) -> list[int]:
        """Slots for `n` new sequences; on failure none is kept."""
        from ..cache import CacheFull
        got = []
        try:
            for _ in range(n):
                got.append(self.engine.slot_alloc())
        except CacheFull:
            self.release(got)
            raise
        return got

    def release(self, slots) -> None:
        for s in slots:
            self.engine.slot_free(s)

    def recorded_steps(self) -> int:
        """Decode steps (by batch size and chunking) that replay a recorded HIP graph."""
        return self.engine.recorded_steps()

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    # -- the step ------------------------------------------------------------------------------
    def step(self, slots, new_tokens, want=None) -> torch.Tensor:
        """Run `new_tokens[i]` for the sequence in `slots[i]`, appended at its current
        length.  `want[i]` lists indices into new_tokens[i]; default: each sequence's last
        token.  Returns float32 logits [sum(len(want[i])), vocab] in the order of the
        sequences and of `want`; the tensor is workspace memory, valid until the next step.
        """
        return self.engine.step(list(slots), new_tokens, want)

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
        return self.engine.step_device_tokens(slots, tokens.contiguous())
