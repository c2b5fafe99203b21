from .pages import PagePool, SlotPool, OutOfPages
from .manager import CacheManager, CacheGroup

__all__ = ["PagePool", "SlotPool", "OutOfPages", "CacheManager", "CacheGroup"]
