from .manager import CacheManager, RequestCache
from .pages import NoFreeSlot, OutOfPages, PagePool, SlotPool
from .storage import KVStorage, StateStorage

__all__ = [
    "CacheManager", "KVStorage", "NoFreeSlot", "OutOfPages", "PagePool", "RequestCache", "SlotPool", "StateStorage",
]
