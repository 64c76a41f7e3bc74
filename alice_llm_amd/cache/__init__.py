from .paged import Cache, CacheError, LayerCache, PageGroup, SlotTable, PAGE_SIZE
