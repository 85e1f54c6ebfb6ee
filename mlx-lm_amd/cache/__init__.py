"""The cache manager: paged keys and values with block tables, and state slots."""

from .manager import CacheManager, KeptPages, OutOfPages, OutOfSlots, RequestCache
from .pages import PagePool

__all__ = ["CacheManager", "KeptPages", "OutOfPages", "OutOfSlots", "PagePool", "RequestCache"]
