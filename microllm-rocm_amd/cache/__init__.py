from .manager import RELEASED, CacheGroup, CacheManager, RequestCache
from .needs import Binding, CacheNeed, PagedBinding, PagedKVNeed, StateBinding, StateNeed
from .pages import OutOfPages, PagePool, SlotPool

__all__ = ["RELEASED", "CacheGroup", "CacheManager", "RequestCache", "Binding", "CacheNeed", "PagedBinding",
           "PagedKVNeed", "StateBinding", "StateNeed", "OutOfPages", "PagePool", "SlotPool"]
