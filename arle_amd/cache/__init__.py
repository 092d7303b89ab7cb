from .manager import (PAGE, CacheManager, NoFreeSlot, PagedNeed, PagedView, PageTensor, StateNeed, StateView,
                      cache_bytes_per_token, pages_for_memory, state_bytes_per_slot)
from .pages import FREED, OutOfPages, PageGroup, PagePool

__all__ = ["CacheManager", "NoFreeSlot", "PagedNeed", "PagedView", "PageTensor", "PAGE", "StateNeed", "StateView",
           "FREED", "OutOfPages", "PageGroup", "PagePool", "cache_bytes_per_token", "pages_for_memory",
           "state_bytes_per_slot"]
