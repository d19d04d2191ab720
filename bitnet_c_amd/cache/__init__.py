from .paged import PAGE, CacheError, CacheFull, PagePool, PagedCache
