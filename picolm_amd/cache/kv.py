"""The cache on the GPU: paged keys and values for each group of layers, a slot for each
live sequence, and fixed-size per-sequence state beside them.

Layout of one KV group: K is [entry][page][kv_head][PAGE_TOKENS][head_dim] and V is kept
transposed, [entry][page][kv_head][head_dim][PAGE_TOKENS] (with a size of its own where a mixer's values
are not as wide as its keys); an entry is one layer call's cache.  A slot's row of the group's page table maps logical page
j (tokens 64j .. 64j+63) to a page; a group that keeps a window of keys maps j modulo its
ring.  picolm's cache is [kv_layer][pos][G*d] for its one sequence, indexed through
kv_layer_ordinal (picolm/model_core.c:734-739, :668-681, :1880-1883); the per-layer-call
entry index here plays that ordinal's role.  State groups are [entry][slot][...] and are
zeroed when a slot is allocated (picolm keeps such state per layer in its arena,
picolm/model.h:303-304).
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

from .slots import PAGE_TOKENS, CacheError, CacheFull, PagedGroupBook, SlotTable, pages_for


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


@dataclass
class CacheSpec:
    kv_groups: list = field(default_factory=list)
    state_groups: list = field(default_factory=list)


WINDOW_STEP_TOKENS = 256     # new tokens of one sequence that a windowed group takes in at once


def window_ring_pages(window: int, step_tokens: int = WINDOW_STEP_TOKENS) -> int:
    """Pages of a slot's ring in a group that keeps `window` keys: enough for the window of the
    first query of a chunk of `step_tokens` new tokens together with the whole chunk, which is
    written before its queries are answered."""
    return pages_for(window - 1 + step_tokens) + 1


class KVGroup:
    def __init__(self, spec: KVGroupSpec, n_pages, n_slots, max_pages, dtype, device):
        self.spec = spec
        self.ring_pages = min(window_ring_pages(spec.window), max_pages) if spec.window > 0 else max_pages
        per_slot = self.ring_pages if spec.window > 0 else max_pages
        n_pages = min(n_pages, n_slots * per_slot)
        self.book = PagedGroupBook(n_pages, n_slots, self.ring_pages if spec.window > 0 else 0)
        n = max(n_pages, 1)
        self.k = torch.zeros((spec.n_entries, n, spec.n_kv_heads, PAGE_TOKENS, spec.head_dim), dtype=dtype, device=device)
        self.v = torch.zeros((spec.n_entries, n, spec.n_kv_heads, spec.value_dim, PAGE_TOKENS), dtype=dtype, device=device)
        self.table_host = torch.zeros((n_slots, max_pages), dtype=torch.int32)
        self.table = torch.zeros((n_slots, max_pages), dtype=torch.int32, device=device)
        self.dirty: set[int] = set()

    def bytes(self) -> int:
        return (self.k.numel() + self.v.numel()) * self.k.element_size()


class Cache:
    """`max_tokens`: the most tokens live sequences hold together, each sequence's count
    rounded up to whole pages; `max_seq_len`: the longest one sequence may get."""

    def __init__(self, spec: CacheSpec, max_tokens: int, max_seq_len: int, dtype: torch.dtype,
                 device, n_slots: int | None = None):
        if max_tokens <= 0 or max_seq_len <= 0:
            raise CacheError("the cache needs a positive token budget and sequence length")
        self.spec = spec
        self.dtype = dtype
        self.device = torch.device(device)
        n_pages = pages_for(max_tokens)
        self.max_seq_len = min(max_seq_len, n_pages * PAGE_TOKENS)
        self.max_pages = pages_for(self.max_seq_len)
        self.n_slots = n_slots if n_slots is not None else n_pages
        self.slots = SlotTable(self.n_slots)
        self.version = 0        # moves whenever a slot or a page changes hands: what was looked up before is stale
        self.kv = [KVGroup(g, n_pages, self.n_slots, self.max_pages, dtype, self.device)
                   for g in spec.kv_groups]
        self.state = [torch.zeros((g.n_entries, self.n_slots, *g.shape), dtype=g.dtype, device=self.device)
                      for g in spec.state_groups]

    # -- slots ---------------------------------------------------------------------------
    def alloc_slot(self) -> int:
        s = self.slots.alloc()
        self.version += 1
        for st in self.state:
            st[:, s].zero_()
        return s

    def free_slot(self, slot: int) -> None:
        self.slots.free(slot)            # raises on a double free before any page moves
        self.version += 1
        for g in self.kv:
            g.book.release(slot)

    def length(self, slot: int) -> int:
        return self.slots.length[slot]

    def reserve(self, slot: int, n_tokens: int) -> None:
        """Give `slot` pages for `n_tokens` tokens in every group, or raise CacheFull and
        change nothing."""
        if not self.slots.is_live(slot):
            raise CacheError(f"slot {slot} is not live")
        if n_tokens > self.max_seq_len:
            raise CacheFull(f"a sequence of {n_tokens} tokens exceeds the cache's {self.max_seq_len}")
        for g in self.kv:
            if g.book.missing(slot, n_tokens) > g.book.pool.n_free:
                raise CacheFull(f"slot {slot} needs {g.book.missing(slot, n_tokens)} more pages, "
                                f"{g.book.pool.n_free} are free")
        for g in self.kv:
            for j, p in g.book.grow(slot, n_tokens):
                g.table_host[slot, j] = p
                g.dirty.add(slot)
                self.version += 1

    def reserve_many(self, slots, lengths) -> None:
        """All or nothing for a whole batch."""
        for s, n in zip(slots, lengths):
            if not self.slots.is_live(s):
                raise CacheError(f"slot {s} is not live")
            if n > self.max_seq_len:
                raise CacheFull(f"a sequence of {n} tokens exceeds the cache's {self.max_seq_len}")
        for g in self.kv:
            need = sum(g.book.missing(s, n) for s, n in zip(slots, lengths))
            if need > g.book.pool.n_free:
                raise CacheFull(f"the batch needs {need} more pages, {g.book.pool.n_free} are free")
        for s, n in zip(slots, lengths):
            self.reserve(s, n)

    def set_length(self, slot: int, n_tokens: int) -> None:
        self.slots.length[slot] = n_tokens

    def flush(self) -> None:
        """Bring the device page tables up to date (rows of slots that got pages)."""
        for g in self.kv:
            for s in sorted(g.dirty):
                row = g.table_host[s]
                if g.table.device.type == "cuda":
                    # through a pinned copy of the row and without waiting for the GPU (a step may
                    # still be running); torch keeps the pinned block until the transfer has run
                    g.table[s].copy_(row.pin_memory(), non_blocking=True)
                else:
                    g.table[s].copy_(row)
            g.dirty.clear()

    def bytes(self) -> int:
        return sum(g.bytes() for g in self.kv) + sum(s.numel() * s.element_size() for s in self.state)

    def free_tokens(self) -> int:
        return min((g.book.pool.n_free for g in self.kv), default=0) * PAGE_TOKENS
