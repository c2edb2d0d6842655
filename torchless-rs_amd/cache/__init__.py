from .cache import PAGE, Cache, KVGroup, KVRequest, StateRequest, pages_for
from .native import CacheFull, CacheMisuse

__all__ = ["PAGE", "Cache", "KVGroup", "KVRequest", "StateRequest", "pages_for", "CacheFull", "CacheMisuse"]
