"""Paged key/value cache: pages, block tables, groups, per-request state slots."""
from .manager import (CacheError, CacheManager, GroupSpec, OutOfPages, PagePool, PositionOverflow,
                      RequestEntry, SlotPool)
from .storage import CacheStorage

__all__ = ["CacheError", "CacheManager", "CacheStorage", "GroupSpec", "OutOfPages", "PagePool",
           "PositionOverflow", "RequestEntry", "SlotPool"]
