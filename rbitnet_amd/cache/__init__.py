from .pages import PAGE_SIZE, FreeList, PageTable, pages_for
from .cache import Cache, KvGroup, LayerCacheView, StateGroup

__all__ = ["PAGE_SIZE", "FreeList", "PageTable", "pages_for", "Cache", "KvGroup", "LayerCacheView", "StateGroup"]
