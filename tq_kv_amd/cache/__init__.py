from .store import PAGE, Cache, CacheFull, Entry

__all__ = ["CacheFull", "PAGE", "Cache", "Entry"]
