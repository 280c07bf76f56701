from .manager import (CacheError, CacheGroup, CacheManager, CacheView, OutOfPages, PagePool, StateSlots, ceil_div,
                      pages_for_memory, windowed_pool_pages)

__all__ = ["CacheError", "CacheGroup", "CacheManager", "CacheView", "OutOfPages", "PagePool", "StateSlots", "ceil_div",
           "pages_for_memory", "windowed_pool_pages"]
