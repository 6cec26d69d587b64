from .pages import CacheFull, CacheMisuse, PagePool, PageTable, SlotTable
from .spec import PAGE_TOKENS, KVNeed, StateNeed, pages_for
from .store import CacheStore, KVLine, StateLine

__all__ = ["CacheFull", "CacheMisuse", "PagePool", "PageTable", "SlotTable", "PAGE_TOKENS", "KVNeed", "StateNeed",
           "pages_for", "CacheStore", "KVLine", "StateLine"]
