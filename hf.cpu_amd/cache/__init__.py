"""The cache: pools of pages with per-request block tables, state slots, device storage."""
from .manager import CacheManager, Group, Held
from .pages import OutOfPages, PagePool
from .storage import CacheStorage, PagedView, StateView

__all__ = ["CacheManager", "CacheStorage", "Group", "Held", "OutOfPages", "PagePool", "PagedView", "StateView"]
