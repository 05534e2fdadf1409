from .manager import CacheManager, CacheView, KVGroup, Sequence, pages_for
from .pages import OutOfPages, PagePool
from .state import OutOfSlots, StateSlots

__all__ = ["CacheManager", "CacheView", "KVGroup", "Sequence", "pages_for", "OutOfPages",
           "PagePool", "OutOfSlots", "StateSlots"]
