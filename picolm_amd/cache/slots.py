"""Host-side bookkeeping of the cache: which pages are free, which slot holds which pages.

Pure Python, no GPU: a slot is one live sequence; it owns pages of PAGE_TOKENS tokens in
every page pool, has a length, and gives everything back when it is freed.  picolm has one
sequence and no slots (its "reset" is a memset, picolm/picolm.c:1391-1392).
"""
from __future__ import annotations

PAGE_TOKENS = 64


class CacheError(RuntimeError):
    pass


class CacheFull(CacheError):
    """Not enough free pages or slots for what was asked."""


def pages_for(n_tokens: int) -> int:
    return (n_tokens + PAGE_TOKENS - 1) // PAGE_TOKENS


class PagePool:
    """A set of page numbers 0..n-1; a page is either free or taken, never both."""

    def __init__(self, n_pages: int):
        if n_pages < 0:
            raise CacheError(f"a pool cannot have {n_pages} pages")
        self.n_pages = n_pages
        self._free = list(range(n_pages - 1, -1, -1))      # pop() hands out low numbers first
        self._taken = [False] * n_pages

    @property
    def n_free(self) -> int:
        return len(self._free)

    def take(self, n: int) -> list[int]:
        if n > len(self._free):
            raise CacheFull(f"{n} pages asked for, {len(self._free)} of {self.n_pages} are free")
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._taken[p] = True
        return out

    def give(self, pages) -> None:
        for p in pages:
            if not 0 <= p < self.n_pages:
                raise CacheError(f"page {p} is not of this pool")
            if not self._taken[p]:
                raise CacheError(f"page {p} is given back twice")
            self._taken[p] = False
            self._free.append(p)


class SlotTable:
    """Slots 0..n-1, each free or live; a live slot has a length."""

    def __init__(self, n_slots: int):
        self.n_slots = n_slots
        self._free = list(range(n_slots - 1, -1, -1))
        self._live = [False] * n_slots
        self.length = [0] * n_slots

    @property
    def n_free(self) -> int:
        return len(self._free)

    def live_slots(self) -> list[int]:
        return [s for s in range(self.n_slots) if self._live[s]]

    def is_live(self, slot: int) -> bool:
        return 0 <= slot < self.n_slots and self._live[slot]

    def alloc(self) -> int:
        if not self._free:
            raise CacheFull(f"all {self.n_slots} slots are live")
        s = self._free.pop()
        self._live[s] = True
        self.length[s] = 0
        return s

    def free(self, slot: int) -> None:
        if not 0 <= slot < self.n_slots:
            raise CacheError(f"slot {slot} does not exist")
        if not self._live[slot]:
            raise CacheError(f"slot {slot} is freed twice")
        self._live[slot] = False
        self.length[slot] = 0
        self._free.append(slot)


class PagedGroupBook:
    """Page ownership of one group of layers: slot -> its pages, in logical order.

    `ring_pages` > 0 bounds how many pages a slot ever holds: logical page j lives in the
    slot's page j % ring_pages (a window of keys); 0 means every key is kept.
    """

    def __init__(self, n_pages: int, n_slots: int, ring_pages: int = 0):
        self.pool = PagePool(n_pages)
        self.ring_pages = ring_pages
        self.pages: list[list[int]] = [[] for _ in range(n_slots)]

    def need(self, n_tokens: int) -> int:
        n = pages_for(n_tokens)
        return min(n, self.ring_pages) if self.ring_pages else n

    def missing(self, slot: int, n_tokens: int) -> int:
        return max(0, self.need(n_tokens) - len(self.pages[slot]))

    def grow(self, slot: int, n_tokens: int) -> list[tuple[int, int]]:
        """Make the slot hold `n_tokens`; returns the (logical index, page) pairs added."""
        k = self.missing(slot, n_tokens)
        if k == 0:
            return []
        first = len(self.pages[slot])
        new = self.pool.take(k)
        self.pages[slot].extend(new)
        return [(first + i, p) for i, p in enumerate(new)]

    def release(self, slot: int) -> None:
        self.pool.give(self.pages[slot])
        self.pages[slot] = []
