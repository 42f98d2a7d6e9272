from .allocator import PAGE_TOKENS, CacheFull, PagePool, SequencePages, SlotTable, pages_for

__all__ = ["PAGE_TOKENS", "CacheFull", "PagePool", "SequencePages", "SlotTable", "pages_for",
           "CacheLayout", "SessionCache"]


def __getattr__(name):  # the storage classes need torch and the parts; load them on demand
    if name in ("CacheLayout", "SessionCache"):
        from . import storage
        return getattr(storage, name)
    raise AttributeError(name)
