from .pages import CacheFull
from .store import PAGE, Cache, KVEntry, StateEntry

__all__ = ["CacheFull", "PAGE", "Cache", "KVEntry", "StateEntry"]
