from .pages import Pool, OutOfPages
from .manager import CacheManager, RequestCache, GroupInfo, NULL_PAGE, first_needed_position, pages_for_spec
from .storage import CacheStorage, LayerCache
from .sizing import CacheTooSmall, cache_groups, memory_budget, page_bytes, size_pools

__all__ = ["Pool", "OutOfPages", "CacheManager", "RequestCache", "GroupInfo", "NULL_PAGE",
           "first_needed_position", "pages_for_spec", "CacheStorage", "LayerCache",
           "CacheTooSmall", "cache_groups", "memory_budget", "page_bytes", "size_pools"]
