from .pages import Pool, OutOfPages
from .manager import CacheManager, RequestCache, GroupInfo, NULL_PAGE, first_needed_position
from .storage import CacheStorage, LayerCache

__all__ = ["Pool", "OutOfPages", "CacheManager", "RequestCache", "GroupInfo", "NULL_PAGE",
           "first_needed_position", "CacheStorage", "LayerCache"]
