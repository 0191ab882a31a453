"""Paged key/value cache with per-request page tables, layer groups and fixed-size state slots."""
from .needs import JointNeed, PagedKvNeed, StateNeed, paged_need, state_need
from .pages import OutOfPages, PageError, PagePool
from .manager import CacheError, CacheManager, PageGroup
from .prefix import PrefixIndex
