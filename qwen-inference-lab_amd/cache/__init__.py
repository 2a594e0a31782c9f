"""Cache: pages, block tables and state slots."""
from .pages import PagePool, CacheFull
from .manager import CacheManager, KVView, PagedView, StateView

__all__ = ['PagePool', 'CacheFull', 'CacheManager', 'KVView', 'PagedView', 'StateView']
