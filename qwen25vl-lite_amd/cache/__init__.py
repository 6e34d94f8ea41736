from .manager import CacheGroupSpec, CacheManager, OutOfPages, OutOfSlots, RequestPages
from .pages import PagePool
from .prefix import RadixPrefixCache
from .storage import KVStorage

__all__ = ["CacheGroupSpec", "CacheManager", "OutOfPages", "OutOfSlots", "RequestPages", "PagePool",
           "RadixPrefixCache", "KVStorage"]
