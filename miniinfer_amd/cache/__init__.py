from .manager import CacheError, CacheManager, LayerCache, OutOfPages, OutOfSlots, PagePool
