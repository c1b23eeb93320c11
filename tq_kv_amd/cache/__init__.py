from .pages import CacheFull, FreeList
from .store import PAGE, Cache, KVEntry, StateEntry

__all__ = ["CacheFull", "FreeList", "PAGE", "Cache", "KVEntry", "StateEntry"]
