from .manager import CacheManager, NoFreeSlot, OutOfPages, RequestCache
from .storage import KVStorage, StateStorage

__all__ = ["CacheManager", "KVStorage", "NoFreeSlot", "OutOfPages", "RequestCache", "StateStorage"]
