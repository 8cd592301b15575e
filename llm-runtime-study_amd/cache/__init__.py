"""Paged key/value cache and per-request state slots."""

from .manager import CacheManager, LayerCache, RequestCache
from .pages import PagePool

__all__ = ["CacheManager", "LayerCache", "PagePool", "RequestCache"]
