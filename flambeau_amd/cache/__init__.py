from .manager import CacheError, CacheManager, GroupSpec, PagePool, RequestCache
