from .manager import FREED, CacheManager, PagedGroup, SequenceCache, StateGroup
from .pages import PageError, PagePool
from .spec import PagedKVSpec, StateSpec

__all__ = ["FREED", "CacheManager", "PagedGroup", "SequenceCache", "StateGroup", "PageError", "PagePool",
           "PagedKVSpec", "StateSpec"]
