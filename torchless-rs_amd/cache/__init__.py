from .cache import PAGE, Cache, KVGroup, KVRequest, StateRequest, pages_for
from .pool import CacheFull, CacheMisuse, FreeList

__all__ = ["PAGE", "Cache", "KVGroup", "KVRequest", "StateRequest", "pages_for", "CacheFull",
           "CacheMisuse", "FreeList"]
