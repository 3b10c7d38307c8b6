from .manager import RELEASED, CacheGroup, CacheManager, RequestCache
from .needs import (Binding, CacheNeed, CompositeBinding, CompositeNeed, LatentBinding, PagedBinding, PagedKVNeed, PagedKeyValueNeed, PagedLatentNeed,
                    StateBinding, StateNeed, flat_bindings, flat_needs)
from .pages import OutOfPages, PagePool, SlotPool

__all__ = ["RELEASED", "CacheGroup", "CacheManager", "RequestCache", "Binding", "CacheNeed", "PagedBinding",
           "PagedKVNeed", "PagedKeyValueNeed", "PagedLatentNeed", "LatentBinding", "CompositeNeed", "CompositeBinding", "flat_needs", "flat_bindings",
           "StateBinding", "StateNeed", "OutOfPages", "PagePool", "SlotPool"]
