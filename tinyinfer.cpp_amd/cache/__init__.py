from .manager import CacheManager, CacheError, OutOfPages, PagePool, PagedGroup
