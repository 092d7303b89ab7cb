from .manager import CacheManager, NoFreeSlot, PagedNeed, PagedView, StateNeed, StateView
from .pages import FREED, OutOfPages, PageGroup, PagePool

__all__ = ["CacheManager", "NoFreeSlot", "PagedNeed", "PagedView", "StateNeed", "StateView", "FREED",
           "OutOfPages", "PageGroup", "PagePool"]
