"""What the cache's bookkeeping says when it is full."""


class CacheFull(RuntimeError):
    """The step needs more pages or slots than are free; nothing was changed."""
