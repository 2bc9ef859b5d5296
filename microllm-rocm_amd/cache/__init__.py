from .manager import RELEASED, CacheGroup, CacheManager, PagedBinding, RequestCache, StateBinding
from .pages import OutOfPages, PagePool, SlotPool

__all__ = ["RELEASED", "CacheGroup", "CacheManager", "PagedBinding", "RequestCache", "StateBinding",
           "OutOfPages", "PagePool", "SlotPool"]
