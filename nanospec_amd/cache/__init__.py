from .manager import RELEASED, CacheManager, GroupSpec, RequestCache
from .pages import PagePool, PoolExhausted, SlotPool

__all__ = ["RELEASED", "CacheManager", "GroupSpec", "RequestCache", "PagePool", "PoolExhausted", "SlotPool"]
