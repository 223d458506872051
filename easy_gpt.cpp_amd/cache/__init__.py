from .manager import CacheManager, RequestCache
from .pages import NoFreeSlot, OutOfPages
from .storage import KVStorage, StateStorage

__all__ = ["CacheManager", "KVStorage", "NoFreeSlot", "OutOfPages", "RequestCache", "StateStorage"]
