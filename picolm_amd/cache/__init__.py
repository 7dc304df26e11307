"""What a model asks of the cache, and the cache's errors.

The cache itself lives in the library (csrc/engine.hip): pages of PAGE_TOKENS tokens, a slot for
each live sequence with a row of the page table, storage per group of layer calls that need the
same kind of keys and values, fixed-size state per sequence beside them.  Layout of one KV group: K
is [entry][page][kv_head][PAGE_TOKENS][head_dim] and V is kept transposed,
[entry][page][kv_head][v_head_dim][PAGE_TOKENS]; an entry is one layer call's cache.  A slot's row
of the group's page table maps logical page j (tokens 64j .. 64j+63) to a page; a group that keeps
a window of keys maps j modulo its ring.  picolm's cache is [kv_layer][pos][G*d] for its one
sequence, indexed through kv_layer_ordinal (picolm/model_core.c:734-739, :668-681, :1880-1883); the
per-layer-call entry index here plays that ordinal's role.  State groups are [entry][slot][...]
and are zeroed when a slot is given out (picolm keeps such state per layer in its arena,
picolm/model.h:303-304).
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

PAGE_TOKENS = 64
WINDOW_STEP_TOKENS = 256     # new tokens of one sequence that a windowed group takes in at once


class CacheError(RuntimeError):
    pass


class CacheFull(CacheError):
    """Not enough free pages or slots for what was asked."""


def pages_for(n_tokens: int) -> int:
    return (n_tokens + PAGE_TOKENS - 1) // PAGE_TOKENS


def window_ring_pages(window: int, step_tokens: int = WINDOW_STEP_TOKENS) -> int:
    """Pages of a slot's ring in a group that keeps `window` keys: enough for the window of the
    first query of a chunk of `step_tokens` new tokens together with the whole chunk, which is
    written before its queries are answered."""
    return pages_for(window - 1 + step_tokens) + 1


@dataclass(frozen=True)
class KVGroupSpec:
    n_entries: int
    n_kv_heads: int
    head_dim: int
    window: int = 0            # 0: all keys are kept; w > 0: the last w keys
    v_head_dim: int = 0        # size of a value where it is not that of a key

    @property
    def value_dim(self) -> int:
        return self.v_head_dim or self.head_dim


@dataclass(frozen=True)
class StateGroupSpec:
    n_entries: int
    shape: tuple
    dtype: torch.dtype = torch.float32

    @property
    def bytes_per_slot(self) -> int:
        n = self.dtype.itemsize
        for s in self.shape:
            n *= int(s)
        return n


@dataclass
class CacheSpec:
    kv_groups: list = field(default_factory=list)
    state_groups: list = field(default_factory=list)


__all__ = ["PAGE_TOKENS", "WINDOW_STEP_TOKENS", "CacheError", "CacheFull", "pages_for", "window_ring_pages",
           "KVGroupSpec", "StateGroupSpec", "CacheSpec"]
