"""The cache: page pools with block tables per request and cache group, and per-request state slots."""

from .manager import CacheManager, GroupSpec
from .pages import CacheLogicError, OutOfPages, PagePool, StateSlots

__all__ = ["CacheManager", "GroupSpec", "CacheLogicError", "OutOfPages", "PagePool", "StateSlots"]
