"""The cache: page pools, block tables, slots."""
from .manager import CacheManager, PagedGroup
from .pool import OutOfPages, PagePool

__all__ = ["CacheManager", "PagedGroup", "OutOfPages", "PagePool"]
