from .paged import CacheError, CacheFull, CacheGroup, KVView, PagedCache, PagePool
