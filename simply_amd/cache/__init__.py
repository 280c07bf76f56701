from .manager import (CacheError, CacheGroup, CacheManager, CacheView, OutOfPages, PagePool, StateSlots, ceil_div)

__all__ = ["CacheError", "CacheGroup", "CacheManager", "CacheView", "OutOfPages", "PagePool", "StateSlots", "ceil_div"]
