from .slots import SlotAllocator, PagePool, CacheError
from .specs import KVSpec, StateSpec
from .cache import Cache, KVGroup, StateGroup, KVView, StateView, PAGE

__all__ = ["SlotAllocator", "PagePool", "CacheError", "KVSpec", "StateSpec", "Cache", "KVGroup",
           "StateGroup", "KVView", "StateView", "PAGE"]
