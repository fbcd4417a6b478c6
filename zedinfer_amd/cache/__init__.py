from .manager import CacheGroup, CacheManager, SequenceCache
from .pages import IdPool, OutOfPages, OutOfSlots, PagePool

__all__ = ["CacheGroup", "CacheManager", "SequenceCache", "IdPool", "OutOfPages", "OutOfSlots", "PagePool"]
