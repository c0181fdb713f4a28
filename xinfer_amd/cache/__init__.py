from .manager import BatchArrays, CacheError, CacheGroup, OutOfPages, PagedCacheManager
