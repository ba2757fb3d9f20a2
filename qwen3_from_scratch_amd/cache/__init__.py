from .manager import CacheManager
from .pages import OutOfPages, PagePool
from .storage import CacheStorage, LayerCacheView

__all__ = ["CacheManager", "CacheStorage", "LayerCacheView", "OutOfPages", "PagePool"]
