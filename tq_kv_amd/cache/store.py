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

The reference keeps one growing tensor pair per layer and one sequence
(src/models/turbo_generic.rs:1606-1618) and resets by position
(src/engine.rs:322-324); lengths after prompt(8), +1, +1 are 8, 9, 10 as in
tq-kv/src/candle_kv.rs:266-299.
"""
import numpy as np
import torch

from ..parts.spec import KVNeed, StateNeed
from .pages import CacheFull, FreeList

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


class KVGroup:
    def __init__(self, need, runs, n_pages, dtype, device):
        self.need = need
        self.runs = list(runs)
        self.pool = FreeList(n_pages, "page")
        shape = (len(self.runs), n_pages, need.n_kv_heads, PAGE, need.head_dim)
        self.keys = torch.zeros(shape, dtype=dtype, device=device)
        self.values = torch.zeros(shape[:3] + (need.head_dim, PAGE), dtype=dtype, device=device)
        self.pages = {}               # slot -> list of page ids, -1 where given back

    def first_needed(self, length):
        """First position a query at or after `length` can still see."""
        if self.need.window is None:
            return 0
        return max(0, length + 1 - self.need.window)

    def missing(self, slot, new_length):
        return max(0, pages_for(new_length) - len(self.pages.get(slot, ())))

    def extend(self, slot, new_length):
        have = self.pages.setdefault(slot, [])
        have.extend(self.pool.take(pages_for(new_length) - len(have)))

    def trim(self, slot, length):
        """Give back the pages whose positions are all out of the window."""
        if self.need.window is None:
            return
        have = self.pages.get(slot, [])
        dead = min(self.first_needed(length) // PAGE, len(have))
        gone = [p for p in have[:dead] if p >= 0]
        if gone:
            self.pool.give_back(gone)
            for i in range(dead):
                have[i] = -1

    def release(self, slot):
        have = self.pages.pop(slot, [])
        self.pool.give_back([p for p in have if p >= 0])


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
        self.slots = FreeList(self.max_slots, "slot")
        self.lengths = [0] * self.max_slots
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
        slot = self.slots.take(1)[0]
        self.lengths[slot] = 0
        for g in self.state_groups:
            g.reset(slot)
        return slot

    def release(self, slot):
        """Give the slot and everything it holds back."""
        self.slots.give_back([slot])
        for g in self.kv_groups:
            g.release(slot)
        self.lengths[slot] = 0

    def length(self, slot):
        return self.lengths[slot]

    # -- one step ---------------------------------------------------------
    def reserve(self, items):
        """items: [(slot, n_new)].  Make room for n_new more positions in every group,
        for all sequences or (CacheFull) for none."""
        for g in self.kv_groups:
            want = 0
            for slot, n_new in items:
                if not self.slots.is_held(slot):
                    raise AssertionError("slot %d is not held" % slot)
                want += g.missing(slot, self.lengths[slot] + n_new)
            if want > g.pool.n_free:
                raise CacheFull("step needs %d more pages of %d positions, %d free of %d"
                                % (want, PAGE, g.pool.n_free, g.pool.n))
        for g in self.kv_groups:
            for slot, n_new in items:
                g.extend(slot, self.lengths[slot] + n_new)

    def commit(self, items):
        """The step has been launched: lengths grow, windows let go of old pages."""
        for slot, n_new in items:
            self.lengths[slot] += n_new
            for g in self.kv_groups:
                g.trim(slot, self.lengths[slot])

    def page_table(self, group, slots):
        """[len(slots), width] int32 of page ids (-1: none) for the sequences of a step."""
        width = max(1, max(len(group.pages.get(s, ())) for s in slots))     # (a group exists only with pages)
        table = np.full((len(slots), width), -1, dtype=np.int32)
        for i, s in enumerate(slots):
            have = group.pages.get(s, ())
            table[i, :len(have)] = have
        return table

    def entry(self, run):
        return self._views[run]

    # -- checks -----------------------------------------------------------
    def tokens_held(self):
        """Positions held by live sequences, each counted up to a multiple of PAGE."""
        return sum(pages_for(self.lengths[s]) * PAGE for s in range(self.max_slots) if self.slots.is_held(s))

    def check(self):
        self.slots.check()
        for g in self.kv_groups:
            g.pool.check()
            held = [p for have in g.pages.values() for p in have if p >= 0]
            if len(held) != len(set(held)):
                raise AssertionError("a page is held by two sequences")
            if len(held) != g.pool.n_held:
                raise AssertionError("%d pages held by sequences, pool says %d" % (len(held), g.pool.n_held))
            for slot in g.pages:
                if not self.slots.is_held(slot):
                    raise AssertionError("free slot %d still holds pages" % slot)
