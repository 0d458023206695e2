from .spec import CacheGroup, CacheLayout, CacheNeed, FixedState, PagedKV
from .pages import CapacityError, PagePool
from .manager import CacheManager, Sequence

__all__ = ["CacheGroup", "CacheLayout", "CacheNeed", "FixedState", "PagedKV", "CapacityError",
           "PagePool", "CacheManager", "Sequence"]
