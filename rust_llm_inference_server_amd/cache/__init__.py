"""The cache: page bookkeeping (native, host only) and the page pools on the device."""
from .manager import CacheManager, GroupSpec, OutOfPages, PageCopy

__all__ = ["CacheManager", "GroupSpec", "OutOfPages", "PageCopy"]
