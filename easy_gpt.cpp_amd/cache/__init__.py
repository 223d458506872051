from .manager import CacheManager, NoFreeSlot, OutOfPages, RequestCache
from .storage import PagedStorage, StateStorage

__all__ = ["CacheManager", "PagedStorage", "NoFreeSlot", "OutOfPages", "RequestCache", "StateStorage"]
