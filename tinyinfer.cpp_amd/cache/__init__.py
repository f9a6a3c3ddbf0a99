from .manager import CacheManager, CacheError, OutOfPages, PagePool, PagedGroup
from .storage import CacheStorage
