from .slots import PAGE_TOKENS, CacheError, CacheFull, PagedGroupBook, PagePool, SlotTable, pages_for
from .kv import (WINDOW_STEP_TOKENS, Cache, CacheSpec, KVGroup, KVGroupSpec, StateGroupSpec,
                 window_ring_pages)

__all__ = ["PAGE_TOKENS", "CacheError", "CacheFull", "PagedGroupBook", "PagePool", "SlotTable",
           "pages_for", "Cache", "CacheSpec", "KVGroup", "KVGroupSpec", "StateGroupSpec",
           "window_ring_pages", "WINDOW_STEP_TOKENS"]
