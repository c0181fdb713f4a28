from .manager import BatchArrays, CacheError, CacheGroup, DecodeStepError, OutOfPages, PagedCacheManager
