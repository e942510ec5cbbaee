"""Paged key/value cache: the manager of pages, block tables and state slots."""
from .manager import CacheError, CacheGroup, CacheManager, OutOfPages

__all__ = ["CacheError", "CacheGroup", "CacheManager", "OutOfPages"]
