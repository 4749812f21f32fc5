"""Paged key/value cache with per-request page tables, layer groups and fixed-size state slots."""
from .needs import PagedKvNeed, StateNeed
from .pages import OutOfPages, PageError, PagePool
from .manager import CacheError, CacheManager, PageGroup
from .prefix import PrefixIndex
