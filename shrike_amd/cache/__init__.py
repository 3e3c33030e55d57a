from .manager import CacheManager, LayerCache, SequenceCache
from .pages import PageError, PagePool, SlotPool

__all__ = ["CacheManager", "LayerCache", "PageError", "PagePool", "SequenceCache", "SlotPool"]
