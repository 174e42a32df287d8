from .pages import CacheFull, PagePool, SlotTable
from .kv_cache import Cache, CacheGroup, KVNeed, StateNeed, check_layout

__all__ = ["CacheFull", "PagePool", "SlotTable", "Cache", "CacheGroup", "KVNeed", "StateNeed", "check_layout"]
