from .block_pool import BlockPool, OutOfBlocks
from .manager import GONE, CacheGroup, CacheManager, CacheView, LayerCache, RequestCache, pages_needed

__all__ = ["BlockPool", "OutOfBlocks", "GONE", "CacheGroup", "CacheManager", "CacheView", "LayerCache",
           "RequestCache", "pages_needed"]
