"""Host-side bookkeeping of the cache: free lists of pages and of slots.

Pure Python, no tensors: what is checked here (nothing lost, nothing held twice,
nothing freed twice) is checked without a GPU.
"""


class CacheFull(RuntimeError):
    """The step needs more pages or slots than are free; nothing was changed."""


class FreeList:
    """A pool of n numbered things (pages or slots), each either free or held."""

    def __init__(self, n, what):
        self.n = int(n)
        self.what = what
        self._free = list(range(self.n - 1, -1, -1))   # pop() hands out 0 first
        self._held = [False] * self.n

    @property
    def n_free(self):
        return len(self._free)

    @property
    def n_held(self):
        return self.n - len(self._free)

    def take(self, count=1):
        if count > len(self._free):
            raise CacheFull("need %d %s(s), %d free of %d" % (count, self.what, len(self._free), self.n))
        out = []
        for _ in range(count):
            i = self._free.pop()
            if self._held[i]:
                raise AssertionError("%s %d handed out twice" % (self.what, i))
            self._held[i] = True
            out.append(i)
        return out

    def give_back(self, items):
        for i in items:
            if not (0 <= i < self.n) or not self._held[i]:
                raise AssertionError("%s %d given back but not held" % (self.what, i))
            self._held[i] = False
            self._free.append(i)

    def is_held(self, i):
        return self._held[i]

    def check(self):
        """Every item is either on the free list once or held, never both."""
        seen = [False] * self.n
        for i in self._free:
            if seen[i]:
                raise AssertionError("%s %d is on the free list twice" % (self.what, i))
            seen[i] = True
            if self._held[i]:
                raise AssertionError("%s %d is both free and held" % (self.what, i))
        for i in range(self.n):
            if not seen[i] and not self._held[i]:
                raise AssertionError("%s %d is lost" % (self.what, i))
