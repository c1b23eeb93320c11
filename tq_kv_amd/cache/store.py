"""The cache as Python sees it: a slot for each live sequence, keys and values for each cached
run of the order, fixed-size state beside them.

Runs of the order with the same need form a group.  A group of pages has storage of its own,

    keys:   [runs in group, pages, key page...]      values: [runs in group, pages, value page...]

(what a page looks like inside is the mixer's business: its need names the two shapes; the
attention kernels' pages are keys [kv heads, PAGE, head_dim] and values [kv heads, head_dim,
PAGE], transposed inside a page) and, per slot, the list of pages that hold the slot's positions.
A group with a window gives pages back as soon as every position in them has left the window.
Mixers with a fixed-size state get one row per slot, zeroed when the slot is taken.

Storage and bookkeeping are the engine library's (csrc/engine/store.cpp, csrc/host_engine.cpp);
the classes here hold its handle and show its memory as torch tensors (views, no copies).

The reference keeps one growing tensor pair per layer and one sequence
(src/models/turbo_generic.rs:1606-1618) and resets by position (src/engine.rs:322-324); lengths
after prompt(8), +1, +1 are 8, 9, 10 as in tq-kv/src/candle_kv.rs:266-299.
"""
import json

import numpy as np

from .. import native
from ..native import CacheFull
from ..parts.spec import need_from_json, need_to_json

PAGE = native.page_size()


def pages_for(n_positions):
    return (n_positions + PAGE - 1) // PAGE


class Entry:
    """What a mixer sees of the cache for one run of the order."""

    def __init__(self, cache, run, group, index, writes):
        self.cache, self.run, self.group, self.writes = cache, run, group, writes
        if isinstance(group, KVGroup):
            self.keys, self.values = group.keys[index], group.values[index]
        else:
            self.state = group.state[index]

    @property
    def need(self):
        return self.group.need


class _PoolView:
    """Free and held counts of a pool of the bookkeeping (the slots, or a group's pages)."""

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
    """slot -> list of page ids (-1 where given back) of a group, read from the bookkeeping."""

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


def _tensor(info, on_gpu, keep):
    return native.view(info["data"], {"float32": native.F32, "bfloat16": native.BF16, "int32": native.I32}[info["dtype"]], info["shape"],
                       on_gpu, keep=keep)


class KVGroup:
    def __init__(self, index, info, book, on_gpu, keep):
        self.index = index
        self.need = need_from_json(info["need"])
        self.runs = list(info["runs"])
        self.n_pages = info["n_pages"]
        self.keys = _tensor(info["keys"], on_gpu, keep)
        self.values = _tensor(info["values"], on_gpu, keep)
        self.pool = _PoolView(book, index)
        self.pages = _PagesView(book, index)

    def first_needed(self, length):
        """First position a query at or after `length` can still see."""
        if self.need.window is None:
            return 0
        return max(0, length + 1 - self.need.window)


class StateGroup:
    def __init__(self, info, on_gpu, keep):
        self.need = need_from_json(info["need"])
        self.runs = list(info["runs"])
        self.state = _tensor(info["state"], on_gpu, keep)


class Cache:
    """Slots, lengths, page tables and storage for all groups of one model.

    needs: for each run of the order its need (KVNeed, StateNeed or None).  cache_of: for each run
    None, or the index of the run whose cache it reads.  max_tokens: positions that live sequences
    may hold together, each sequence counted up to a multiple of PAGE.  An engine's cache is shown
    through the same class (of_engine).
    """

    def __init__(self, needs, cache_of, max_tokens, max_slots, dtype, device, _engine=None):
        import torch
        import weakref
        self._lib = native.library()
        self._engine = weakref.proxy(_engine) if _engine is not None else None      # the engine owns its cache, not the other way round
        self.device = torch.device(device)
        self.on_gpu = self.device.type == "cuda"
        if _engine is None:
            co = np.ascontiguousarray([-1 if c is None else int(c) for c in cache_of], dtype=np.int32)
            self.handle = native.handle(self._lib.tqe_store_new(
                native.enc(json.dumps([need_to_json(n) for n in needs])), co.ctypes.data_as(native._I32P), len(needs), int(max_tokens),
                int(max_slots), native.dtype_code(dtype), 1 if self.on_gpu else 0))
            info = native.parsed(self._lib.tqe_store_describe(self.handle))
            book = self._lib.tqe_store_cache(self.handle)
        else:
            self.handle = None
            info = native.parsed(self._lib.tqe_engine_describe(_engine.handle))
            book = self._lib.tqe_engine_cache(_engine.handle)
        self.holds_pages = bool(info["holds_pages"])
        self.n_pages = info["n_pages"]
        self.max_slots = info["max_slots"]
        self.native = native.NativeCache(self.max_slots, [(g["n_pages"], g["need"].get("window")) for g in info["page_groups"]], handle=book)
        self.kv_groups = [KVGroup(i, g, self.native, self.on_gpu, None) for i, g in enumerate(info["page_groups"])]
        self.state_groups = [StateGroup(g, self.on_gpu, None) for g in info["state_groups"]]
        self.slots = _PoolView(self.native, -1)
        self._views = {}
        n_runs = len(needs)
        for run in range(n_runs):
            if needs[run] is None:
                self._views[run] = None
                continue
            owner = run if cache_of[run] is None else cache_of[run]
            for group in self.kv_groups + self.state_groups:
                if owner in group.runs:
                    self._views[run] = Entry(self, run, group, group.runs.index(owner), cache_of[run] is None)

    @classmethod
    def of_engine(cls, engine, needs, cache_of, dtype, device):
        return cls(needs, cache_of, 0, 0, dtype, device, _engine=engine)

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            self.kv_groups = self.state_groups = []
            self._lib.tqe_store_free(h)

    # -- slots ------------------------------------------------------------
    def acquire(self):
        """A free slot with length 0 and zeroed state."""
        import ctypes
        if self._engine is not None:
            return self._engine.open()
        slot = ctypes.c_int32(-1)
        native.check(self._lib.tqe_store_acquire(self.handle, ctypes.byref(slot), native.current_stream() if self.on_gpu else None))
        return slot.value

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
