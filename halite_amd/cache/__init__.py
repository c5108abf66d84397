from .manager import CacheManager
from .pages import CacheGroup, LayerPages, NoSpace, PagePool
from .slots import NoSlot, SlotAllocator, StateStore

__all__ = [
    "CacheGroup", "CacheManager", "LayerPages", "NoSlot", "NoSpace", "PagePool",
    "SlotAllocator", "StateStore",
]
