from .manager import CacheManager, PagedView, StateView, StepTables
from .pages import FreeList, KVCapacityError
from .spec import PagedKVSpec, StateSpec

__all__ = ["CacheManager", "PagedView", "StateView", "StepTables", "FreeList", "KVCapacityError",
           "PagedKVSpec", "StateSpec"]
