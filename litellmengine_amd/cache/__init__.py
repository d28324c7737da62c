from .manager import CacheGroup, CacheManager, GroupSizes, LayerCache
from .page_pool import OutOfPages, PagePool

__all__ = ["CacheGroup", "CacheManager", "GroupSizes", "LayerCache", "OutOfPages", "PagePool"]
