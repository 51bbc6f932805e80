from .manager import CacheManager, KVView, StateView
from .needs import FixedState, PagedKV
from .pages import CacheError, OutOfPages, PagePool

__all__ = ["CacheManager", "KVView", "StateView", "FixedState", "PagedKV", "CacheError", "OutOfPages", "PagePool"]
