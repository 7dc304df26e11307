"""A model with its cache and workspace: the object that generation and trace replay drive.

`begin` gives each new sequence a slot, `step` runs a batch of them from the cache and
returns logits at the wanted rows, `release` gives slots and pages back.  A step never
runs tokens it was not given: the prompt once, then one token each.
"""
from __future__ import annotations

import torch

from ..cache import Cache, CacheFull
from ..parts.base import Workspace
from .batch import StepBatch, StepError
from .model import DecoderModel


class Session:
    def __init__(self, model: DecoderModel, max_tokens: int, max_seq_len: int | None = None,
                 n_slots: int | None = None):
        if model.runtime is None:
            raise StepError("the model has no weights loaded")
        self.model = model
        self.cache: Cache = model.new_cache(max_tokens, max_seq_len, n_slots)
        self.workspace = Workspace(model.runtime.device)
        self.vocab_size = model.head.V

    # -- slots -------------------------------------------------------------------------------
    def begin(self, n: int = 1) -> list[int]:
        """Slots for `n` new sequences; on failure none is kept."""
        got = []
        try:
            for _ in range(n):
                got.append(self.cache.alloc_slot())
        except CacheFull:
            for s in got:
                self.cache.free_slot(s)
            raise
        return got

    def release(self, slots) -> None:
        for s in slots:
            self.cache.free_slot(s)

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
        for s in slots:
            if not self.cache.slots.is_live(s):
                raise StepError(f"slot {s} is not live")
        if want is None:
            want = [[len(t) - 1] for t in new_tokens]
        pos0 = [self.cache.length(s) for s in slots]
        n_new = [len(t) for t in new_tokens]
        batch = StepBatch(slots, pos0, new_tokens, want, self.vocab_size, self.model.runtime.device)
        self.cache.reserve_many(slots, [p + n for p, n in zip(pos0, n_new)])
        self.cache.flush()
        logits = self.model.step(self.cache, batch, self.workspace)
        for s, p, n in zip(slots, pos0, n_new):
            self.cache.set_length(s, p + n)
        return logits
