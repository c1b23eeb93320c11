"""The cache: a slot for each live sequence, keys and values for each cached run of
the order, fixed-size state beside them.

Runs of the order with the same need (same kv heads, head size and window) form a
group.  A group has storage of its own: one pool of pages of PAGE positions,

    keys:   [runs in group, pages, kv heads, PAGE, head_dim]
    values: [runs in group, pages, kv heads, head_dim, PAGE]   (transposed inside a page:
            the attention kernels read 8 consecutive positions of one element at once)

and, per slot, the list of pages that hold the slot's positions.  A group with a
window gives pages back as soon as every position in them has left the window; a
group without keeps them until the slot is released.  Mixers with a fixed-size
state get one float32 row per slot, zeroed when the slot is taken.

The bookkeeping (free slots, lengths, page lists) is the engine's host library's
(csrc/host_engine.cpp behind the C boundary csrc/tq_engine.h); the classes here own the
storage tensors and show the bookkeeping to Python.

The reference keeps one growing tensor pair per layer and one sequence
(src/models/turbo_generic.rs:1606-1618) and resets by position
(src/engine.rs:322-324); lengths after prompt(8), +1, +1 are 8, 9, 10 as in
tq-kv/src/candle_kv.rs:266-299.
"""
import numpy as np
import torch

from .. import native
from ..parts.spec import KVNeed, StateNeed
from .pages import CacheFull

PAGE = 64


def pages_for(n_positions):
    return (n_positions + PAGE - 1) // PAGE


class KVEntry:
    """What an attention-like mixer sees of the cache for one run of the order."""

    def __init__(self, group, index, writes):
        self.group = group
        self.keys = group.keys[index]
        self.values = group.values[index]
        self.writes = writes          # False: reads another run's cache

    @property
    def need(self):
        return self.group.need


class StateEntry:
    """What a mixer with fixed-size state sees: state[slot] is its sequence's row."""

    def __init__(self, group, index, writes):
        self.group = group
        self.state = group.state[index]
        self.writes = writes


class _PoolView:
    """Free and held counts of a pool of the native cache (the slots, or a group's pages)."""

    def __init__(self, cache, group):
        self._cache, self._group = cache, group

    @property
    def n(self):
        return self._cache.counts(self._group)[1]

    @property
    def n_free(self):
        return self._cache.counts(self._group)[0]

    @property
    def n_held(self):
        free, total = self._cache.counts(self._group)
        return total - free

    def is_held(self, i):
        if self._group != -1:
            raise TypeError("only slots can be asked for one by one")
        return self._cache.is_held(i)


class _PagesView:
    """slot -> list of page ids (-1 where given back) of a group, read from the native cache."""

    def __init__(self, cache, group):
        self._cache, self._group = cache, group

    def get(self, slot, default=None):
        have = self._cache.pages(self._group, slot)
        return default if have is None else have

    def __getitem__(self, slot):
        have = self._cache.pages(self._group, slot)
        if have is None:
            raise KeyError(slot)
        return have

    def __contains__(self, slot):
        return self._cache.pages(self._group, slot) is not None

    def __iter__(self):
        return (s for s in range(self._cache.max_slots) if s in self)

    def values(self):
        return [self[s] for s in self]


class KVGroup:
    def __init__(self, need, runs, n_pages, dtype, device):
        self.need = need
        self.runs = list(runs)
        self.n_pages = n_pages
        shape = (len(self.runs), n_pages, need.n_kv_heads, PAGE, need.head_dim)
        self.keys = torch.zeros(shape, dtype=dtype, device=device)
        self.values = torch.zeros(shape[:3] + (need.head_dim, PAGE), dtype=dtype, device=device)
        self.pool = self.pages = None      # views of the native bookkeeping, set by the cache

    def first_needed(self, length):
        """First position a query at or after `length` can still see."""
        if self.need.window is None:
            return 0
        return max(0, length + 1 - self.need.window)


STATE_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


class StateGroup:
    def __init__(self, need, runs, n_slots, device):
        self.need = need
        self.runs = list(runs)
        if need.dtype not in STATE_DTYPES:
            raise TypeError("state of kind %r (known: %s)" % (need.dtype, ", ".join(sorted(STATE_DTYPES))))
        self.state = torch.zeros((len(self.runs), n_slots) + tuple(need.shape),
                                 dtype=STATE_DTYPES[need.dtype], device=device)

    def reset(self, slot):
        self.state[:, slot].zero_()


class Cache:
    """Slots, lengths, page tables and storage for all groups of one model.

    needs: for each run of the order its need (KVNeed, StateNeed or None).
    cache_of: for each run None, or the index of the run whose cache it reads.
    max_tokens: positions that live sequences may hold together, each sequence
    counted up to a multiple of PAGE.
    """

    def __init__(self, needs, cache_of, max_tokens, max_slots, dtype, device):
        # pages bound the cache only where some run keeps keys and values: a model whose runs all
        # keep fixed-size state (or nothing) is bounded by its slots alone
        self.holds_pages = any(isinstance(need, KVNeed) and cache_of[run] is None for run, need in enumerate(needs))
        if self.holds_pages and max_tokens < PAGE:
            raise ValueError("max_tokens must be at least %d, got %d" % (PAGE, max_tokens))
        self.n_pages = max_tokens // PAGE if self.holds_pages else 0
        self.max_slots = max(1, min(int(max_slots), self.n_pages)) if self.holds_pages else max(1, int(max_slots))
        self.device = device
        self.kv_groups = []
        self.state_groups = []
        self._entry = {}              # run index -> (group, index within group)
        by_need = {}
        for run, need in enumerate(needs):
            if need is None or cache_of[run] is not None:
                continue
            by_need.setdefault(need, []).append(run)
        for need, runs in by_need.items():
            if isinstance(need, KVNeed):
                group = KVGroup(need, runs, self.n_pages, dtype, device)
                self.kv_groups.append(group)
            elif isinstance(need, StateNeed):
                group = StateGroup(need, runs, self.max_slots, device)
                self.state_groups.append(group)
            else:
                raise TypeError("unknown cache need %r" % (need,))
            for i, run in enumerate(runs):
                self._entry[run] = (group, i)
        if len(self.kv_groups) > native.MAX_GROUPS:
            raise ValueError("%d groups of cached runs, the engine's library takes %d" % (len(self.kv_groups), native.MAX_GROUPS))
        # the bookkeeping: free slots, lengths, page lists
        self.native = native.NativeCache(self.max_slots, [(g.n_pages, g.need.window) for g in self.kv_groups])
        self.slots = _PoolView(self.native, -1)
        for i, g in enumerate(self.kv_groups):
            g.index = i
            g.pool = _PoolView(self.native, i)
            g.pages = _PagesView(self.native, i)
        self._views = {}
        for run, need in enumerate(needs):
            src = cache_of[run]
            if need is None:
                self._views[run] = None
                continue
            owner = run if src is None else src
            if owner not in self._entry:
                raise ValueError("run %d reads the cache of run %d, which keeps none" % (run, owner))
            group, i = self._entry[owner]
            if src is not None and group.need != need:
                raise ValueError("run %d needs %r but run %d's cache is %r" % (run, need, owner, group.need))
            cls = KVEntry if isinstance(group, KVGroup) else StateEntry
            self._views[run] = cls(group, i, writes=(src is None))

    # -- slots ------------------------------------------------------------
    def acquire(self):
        """A free slot with length 0 and zeroed state."""
        slot = self.native.acquire()
        for g in self.state_groups:
            g.reset(slot)
        return slot

    def release(self, slot):
        """Give the slot and everything it holds back."""
        self.native.release(slot)

    def length(self, slot):
        return self.native.length(slot)

    @property
    def lengths(self):
        return [self.native.length(s) for s in range(self.max_slots)]

    # -- one step ---------------------------------------------------------
    def reserve(self, items):
        """items: [(slot, n_new)].  Make room for n_new more positions in every group,
        for all sequences or (CacheFull) for none."""
        self.native.reserve(items)

    def commit(self, items):
        """The step has been launched: lengths grow, windows let go of old pages."""
        self.native.commit(items)

    def page_table(self, group, slots):
        """[len(slots), width] int32 of page ids (-1: none) for the sequences of a step."""
        lists = [group.pages.get(s, ()) for s in slots]
        width = max(1, max(len(have) for have in lists))
        table = np.full((len(slots), width), -1, dtype=np.int32)
        for i, have in enumerate(lists):
            table[i, :len(have)] = have
        return table

    def entry(self, run):
        return self._views[run]

    # -- checks -----------------------------------------------------------
    def tokens_held(self):
        """Positions held by live sequences, each counted up to a multiple of PAGE."""
        return sum(pages_for(self.native.length(s)) * PAGE for s in range(self.max_slots) if self.native.is_held(s))

    def check(self):
        """Nothing lost, held twice or freed twice (AssertionError with the finding)."""
        self.native.check()
