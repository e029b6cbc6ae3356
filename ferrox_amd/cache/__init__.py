from .manager import CacheManager, PagePool, StateSlots

__all__ = ["CacheManager", "PagePool", "StateSlots"]
