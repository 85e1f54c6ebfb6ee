"""The cache manager: paged keys and values with block tables, and state slots."""

from .manager import CacheManager, OutOfPages, OutOfSlots, RequestCache
from .pages import PagePool

__all__ = ["CacheManager", "OutOfPages", "OutOfSlots", "PagePool", "RequestCache"]
