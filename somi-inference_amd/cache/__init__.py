"""Paged cache pools, block tables and state slots."""

from .manager import RELEASED, CacheManager, PagedGroup, RequestCache
from .pool import CacheError, OutOfPages, PagePool

__all__ = ["CacheError", "CacheManager", "OutOfPages", "PagePool", "PagedGroup", "RELEASED", "RequestCache"]
