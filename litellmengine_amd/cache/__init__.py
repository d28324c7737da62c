from .manager import CacheGroup, CacheManager, LayerCache
from .page_pool import OutOfPages, PagePool

__all__ = ["CacheGroup", "CacheManager", "LayerCache", "OutOfPages", "PagePool"]
