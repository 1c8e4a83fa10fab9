from .manager import CacheError, CacheManager, GroupSpec, OutOfPages, PageGroup, PagePool
